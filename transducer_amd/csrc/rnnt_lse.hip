// Log-normaliser LN[t,u] = log sum_v exp(E[t,v] + P[u,v])  (transducer/torch_binding.py:35-40,
// transducer/test.h:51-80) for gfx950, streaming form on the bf16 matrix cores.
//
// With row maxima mE[t], mP[u] taken out, the sum is the contraction  sum_v X[t,v] * Y[u,v],
// X = exp(E - mE), Y = exp(P - mP), both in (0, 1].  Each fp32 factor is split exactly into three
// bf16 pieces and six piece products are accumulated in fp32 (rnnt_split.h), which keeps fp32
// accuracy at 3/8 of the fp32 matrix-instruction time and leaves the vector ALUs to the exps.
//
//  * Y is small (B*U*V) and used by every frame tile, so it is prepared ONCE: yplanes_kernel
//    writes its three pieces in the matrix instruction's own operand order
//        [b][block of 32 u][step of 16 v][piece][lane 0..63][8 x bf16]
//    and the contraction reads a fragment with one perfectly coalesced 16-byte load per lane,
//    no LDS and no arithmetic.  Steps past V hold zeros, which also takes care of the tail of
//    the reduction: X only has to be finite there.
//  * X is large (B*T*V) and used once: a workgroup turns a 128 x 32 slab of E into the three
//    pieces on its way into LDS (16-byte slots, XOR-swizzled so that the 16-byte fragment reads
//    of eight consecutive rows and the staging writes both spread over all banks).
//  * A wavefront owns one block of 32 label positions and all 128 frames of the tile: four
//    accumulators, 24 matrix instructions per step of 16 v.
//  * The matrix instruction aligns its products to the accumulator and TRUNCATES what falls
//    below the accumulator's last bit, so a long running sum drifts low by a fraction of an ulp
//    per instruction (3750 instructions per output at V = 10000: about 2^-16 relative, measured).
//    Every kFlush slabs the running sums are therefore added (vector ALU, round to nearest) into
//    a second set of accumulators and restarted: the truncation then acts on a sum that is
//    V / (32 kFlush) times smaller.
//  * No separate pass over E for its row maxima: any reference m[t] works in X = exp(E - m[t]) as
//    long as it is taken back out at the end, so a row starts with the maximum of its first 32
//    values and keeps it unless a later value exceeds it by more than kSlack (then the sums of
//    that row are multiplied by exp(old - new) once; rare).  The final reference is written out
//    as mE[t] for the gradient kernels, which only need it to be consistent with LN.
//  * Workgroups are renumbered so that all frame tiles of one utterance run on the same XCD
//    (workgroup ids are dealt round-robin to the 8 XCDs) and share its L2 copy of Y[b].
#include <type_traits>

#include "rnnt_internal.h"
#include "rnnt_io.h"
#include "rnnt_split.h"

namespace rnnt {

namespace {

constexpr int kRowsMax = 128;  // frames per workgroup tile (64 where the grid would be small)
constexpr int kSlice = 32;    // v per LDS slab (two matrix-instruction steps)
constexpr int kFlush = 8;     // slabs between two flushes of the running sums
constexpr float kSlack = 40.0f;  // a row's reference moves when a value tops it by more than this
constexpr float kLowest = -1.0e30f;  // stands in for a reference of -inf (a slab of -inf scores)

__device__ inline int mfma_row(int r, int h) { return 8 * (r >> 2) + 4 * h + (r & 3); }

// Value of lane ^ 1 / lane ^ 2 within each group of four lanes: a DPP move, no LDS round trip.
__device__ inline float quad_xor1(float x) {
  return __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(x), 0xB1, 0xf, 0xf, true));
}
__device__ inline float quad_xor2(float x) {
  return __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(x), 0x4E, 0xf, 0xf, true));
}

// Maxima as single instructions.  fmaxf on values that come straight from memory makes the
// compiler quiet possible signalling NaNs first (one extra instruction per operand); the
// instructions themselves already return the other operand for a NaN.
__device__ inline float vmax3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
__device__ inline float vmax2(float a, float b) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}

// a + b + c rounded once: the two partial sums are carried with their rounding errors (two
// error-free additions; this file is compiled without contraction or reassociation), so the
// log-normaliser's epilogue log(sum) + mE + mP adds half an ulp to the error of the logarithm
// instead of three half ulps.
// `tiny`: a fourth term far below the others' last bits, added to the carried errors.
__device__ inline float add3(float a, float b, float c, float tiny = 0.0f) {
  const float s = b + c, bv = s - b;
  const float s_err = (b - (s - bv)) + (c - bv);
  const float r = a + s, av = r - a;
  const float r_err = (a - (r - av)) + (s - av);
  return r + ((r_err + s_err) + tiny);
}

// X = exp(e - m) for the 32 values of a slab that share the row's reference m.  With m log2(e)
// formed once per row and slab, an exponential is one fused multiply-add and one v_exp_f32
// instead of a subtraction, a multiplication and the v_exp_f32.  The rounding of that product
// moves the reference actually used to m' = fl(m log2 e) / log2 e: the same for every value of
// the row, so it does not touch the sum's accuracy, and the write-out adds m' - m back
// (reference_shift) so that the log-normaliser does not carry it either.
constexpr float kLog2e = 1.44269504088896340736f;
__device__ inline float reference_shift(float m) {
  const float ml = m * kLog2e;
  const float lost = __builtin_fmaf(m, kLog2e, -ml);  // m log2 e - fl(m log2 e), exactly
  return -lost * (1.0f / kLog2e);
}

// 16-byte slot of (row, c8 = which eight of the slab's 32 v) inside a piece plane
__device__ inline int xslot(int row, int c8) { return row * 4 + (c8 ^ ((row >> 2) & 3)); }

inline int y_ublocks(const Dims& d) { return (d.U + 31) / 32; }
inline int y_steps(const Dims& d) { return 2 * ((d.V + kSlice - 1) / kSlice); }

// ------------------------------------------------------------------ Y pieces
// One thread per (u, eight consecutive v).  vec = rows of P start 16-byte aligned (V a multiple
// of 4 for fp32, of 8 for bf16, and P aligned).
template <typename TIO>
__global__ __launch_bounds__(256) void yplanes_kernel(const TIO* __restrict__ P,
                                                      const float* __restrict__ mP,
                                                      uint4* __restrict__ Yp,
                                                      const int* __restrict__ labLen, Dims d,
                                                      int nub, int nks, int vec4) {
  const int b = blockIdx.z, ub = blockIdx.y, ks = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (ks >= nks) return;
  const int lane = threadIdx.x & 63, l32 = lane & 31, h = lane >> 5;
  int Ub = d.U;
  if (labLen) Ub = min(max(labLen[b], 0) + 1, d.U);
  if (32 * ub >= Ub) return;  // a block of rows past the utterance is never read
  const int u = 32 * ub + l32, v0 = 16 * ks + 8 * h;
  float y[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) y[i] = 0.0f;
  if (u < Ub) {
    const TIO* row = P + ((size_t)b * d.U + u) * d.V;
    const float m = mP[(size_t)b * d.U + u];
    if (v0 < d.V) {
      float e[8];  // clamped loads repeat values of the row; masked below
      if (vec4) expand(load8(row, v0, d.V), e);
      else expand(load8_any(row, v0, d.V), e);
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (v0 + i < d.V) y[i] = __expf(e[i] - m);
    }
  }
  const Frag3 f = split8(y);
  uint4* dst = Yp + (((size_t)b * nub + ub) * nks + ks) * 3 * 64 + lane;
  dst[0] = f.h;
  dst[64] = f.m;
  dst[128] = f.l;
}

// ------------------------------------------------------------------ contraction
// kRows frames x 128 label positions per workgroup.  kWaves = 4: a wavefront owns one block of
// 32 label positions and all kRows frames (four accumulators at 128 frames, two at 64).
// kWaves = 8: two wavefronts share a block, half the frames each (half the registers, twice the
// wavefronts to hide each other's staging).  64 frames for grids that 128 would leave below one
// workgroup per CU (each workgroup walks all columns, so a small grid is a long walk on a few
// CUs: B=32 T=400 U=101 V=4096 0.25 -> 0.18 ms, B=8 T=2000 U=101 V=2000 0.147 -> 0.096).
// kVec: rows start 16-byte aligned and hold a multiple of the vector width, so a thread's eight
// values are one or two 16-byte loads; otherwise they are fetched one by one.
template <int kWaves, typename TIO, bool kVec, int kRows>
__global__ __launch_bounds__(64 * kWaves, kWaves / 2) void lse_stream_kernel(
    const TIO* __restrict__ E, float* __restrict__ mE, const float* __restrict__ mP,
    const uint4* __restrict__ Yp, float* __restrict__ LN, const int* __restrict__ inLen,
    const int* __restrict__ labLen, Dims d, int ttiles, int utiles, int total, int nub, int nks,
    const int* __restrict__ labels, float* __restrict__ elS, float* __restrict__ ebv,
    float* __restrict__ lnS) {
  constexpr int kThreads = 64 * kWaves;
  constexpr int MB = kRows / 8 / kWaves;   // 32-frame blocks per wavefront
  constexpr int NR = 4 * kRows / kThreads;  // (row, eight v) items a thread stages per slab
  constexpr int kSlots = kRows * 4;        // 16-byte slots per piece plane: 4 per row
  static_assert(MB >= 1 && NR >= 1, "a tile gives every wavefront a frame block and every thread a row");
  __shared__ uint4 Xs[2][3][kSlots];
  __shared__ float scale[kRows];  // pending factor for a row's sums (1 when its reference stood)
  __shared__ float mfin[kRows];   // final references, for the write-out
  __shared__ int moved;           // some row's reference moved while the last slab was staged
  __shared__ int labs[1025];      // columns to pick: the utterance's labels, then the blank
  __shared__ short order[1025];   // their indices sorted by column
  __shared__ int scol[1025];      // and the columns in that order
  // XCD-aware renumbering: physical id n runs on XCD n % 8
  const int n = blockIdx.x, per_xcd = gridDim.x >> 3;
  const int logical = (n & 7) * per_xcd + (n >> 3);
  if (logical >= total) return;
  const int b = logical / (ttiles * utiles);
  const int rem = logical - b * (ttiles * utiles);
  const int t0 = (rem % ttiles) * kRows, u0 = (rem / ttiles) * 128;
  int Tb, Ub;
  utt_extent(inLen, labLen, b, d.T, d.U, Tb, Ub);
  float* LNb = LN + (size_t)b * d.T * d.U;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, h = lane >> 5;

  // lnS given: LN goes straight into the lattice walk's skewed plane (valid cells only, as a
  // transposing copy would leave it) and the row-major array is not written at all.
  if (t0 >= Tb || u0 >= Ub) {
    if (lnS == nullptr)
      for (int e = tid; e < kRows * 128; e += kThreads) {
        const int t = t0 + e / 128, u = u0 + e % 128;
        if (t < d.T && u < d.U) LNb[(size_t)t * d.U + u] = 0.0f;
      }
    if (t0 >= Tb)  // frames past the utterance report a reference of 0
      for (int r = tid; r < kRows; r += kThreads)
        if (t0 + r < d.T) mE[(size_t)b * d.T + t0 + r] = 0.0f;
    return;
  }
  for (int r = tid; r < kRows; r += kThreads) scale[r] = 1.0f;
  if (tid == 0) moved = 0;
  // Picks: the lattice recursions need E[t, blank] and E[t, label_u] in the skewed planes.  Every
  // element of the tile's rows passes through the staging registers exactly once, so the thread
  // that holds a wanted column copies it out then (first label tile only; ebv == nullptr: off;
  // without labels only the blank column is wanted and elS is not touched).
  const bool picking = ebv != nullptr && u0 == 0;
  const int nlab = (picking && labels != nullptr) ? min(Ub - 1, 1024) : 0;
  const int npick = picking ? nlab + 1 : 0;  // entry nlab is the blank column
  for (int u = tid; u < npick; u += kThreads)
    labs[u] = u < nlab ? label_at(labels, d, b, u) : d.blank;
  __syncthreads();
  // rank every entry by (column, index): the slabs come by in column order, so one cursor into
  // the sorted list tells each slab which columns to copy, at one LDS read per slab
  for (int u = tid; u < npick; u += kThreads) {
    const int c = labs[u];
    int rank = 0;
    for (int w = 0; w < npick; ++w) {
      const int cw = labs[w];
      rank += (cw < c || (cw == c && w < u)) ? 1 : 0;
    }
    order[rank] = (short)u;
    scol[rank] = c;
  }
  int cursor = 0;   // uniform: entries before it have been copied
  int ncol = -1;    // column and index of entry `cursor`, -1 past the last: read one entry ahead, so
  int nu = 0;       // that a slab without a pick costs one scalar comparison
  auto next_pick = [&]() {
    const bool more = cursor < npick;
    const int c = more ? scol[cursor] : -1, u = more ? order[cursor] : 0;
    ncol = __builtin_amdgcn_readfirstlane(c);
    nu = __builtin_amdgcn_readfirstlane(u);
  };

  // staging: thread -> rows srow (+ 64 with four wavefronts) of the tile, v = slab start +
  // 8*c8 .. +7.  Rows past the utterance repeat its last frame, columns past V repeat earlier
  // ones of the row (its last group of four or eight, or its last element when the values are
  // fetched one by one): finite values that meet zeros in Y or are dropped on the way out.
  const int srow = tid >> 2, c8 = tid & 3;
  const TIO* px[NR];
  float mx[NR];  // the row's reference; the four threads that share a row always agree on it
  int slot[NR];
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int row = srow + (kThreads / 4) * i;
    const int t = min(t0 + row, Tb - 1);
    px[i] = E + ((size_t)b * d.T + t) * d.V;
    mx[i] = kLowest;
    slot[i] = xslot(row, c8);
  }
  struct XRegs { Raw8<TIO> x[NR]; };
  auto fetch = [&](int k0) -> XRegs {
    XRegs r;
#pragma unroll
    for (int i = 0; i < NR; ++i)
      r.x[i] = kVec ? load8(px[i], k0 + 8 * c8, d.V) : load8_any(px[i], k0 + 8 * c8, d.V);
    return r;
  };
  // copies column `col` (which lies in the slab held in r) of this thread's rows to the blank
  // vector (nu_plane < 0: dst[t]) or to label position nu_plane of the skewed plane dst
  auto pick = [&](const XRegs& r, int col, float* dst, int nu_plane) {
    if (c8 != ((col & 31) >> 3)) return;
    const int e = col & 7;  // uniform
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      // element e of the eight this thread holds, selected with masks: an indexed access would
      // send the staging registers through scratch memory on every slab
      const unsigned k0 = e == 0 ? ~0u : 0u, k1 = e == 1 ? ~0u : 0u, k2 = e == 2 ? ~0u : 0u,
                     k3 = e == 3 ? ~0u : 0u, k4 = e == 4 ? ~0u : 0u, k5 = e == 5 ? ~0u : 0u,
                     k6 = e == 6 ? ~0u : 0u, k7 = e == 7 ? ~0u : 0u;
      float x[8];
      expand(r.x[i], x);
      const float v = __uint_as_float(
          (__float_as_uint(x[0]) & k0) | (__float_as_uint(x[1]) & k1) |
          (__float_as_uint(x[2]) & k2) | (__float_as_uint(x[3]) & k3) |
          (__float_as_uint(x[4]) & k4) | (__float_as_uint(x[5]) & k5) |
          (__float_as_uint(x[6]) & k6) | (__float_as_uint(x[7]) & k7));
      const int t = t0 + srow + (kThreads / 4) * i;
      if (t < Tb) dst[nu_plane < 0 ? (size_t)t : plane_at(d, b, nu_plane, t + nu_plane)] = v;
    }
  };
  auto picks = [&](const XRegs& r, int kslab) {
    while ((ncol >> 5) == kslab) {  // uniform
      if (nu == nlab) pick(r, ncol, ebv + (size_t)b * d.Tp + d.Eo, -1);
      else pick(r, ncol, elS, nu);
      ++cursor;
      next_pick();
    }
  };
  auto stash = [&](int buf, const XRegs& r, bool first, int kslab) {
    // maximum of each row's 32 values of this slab (values past V repeat earlier ones); taken
    // before the picks so that the loads are waited for here and not inside the pick loop
    float lm[NR];
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      float e[8];
      expand(r.x[i], e);
      float m = vmax3(e[0], e[1], e[2]);
      m = vmax3(m, e[3], e[4]);
      m = vmax2(m, vmax3(e[5], e[6], e[7]));
      m = vmax2(m, quad_xor1(m));  // the four threads of a row are one quad of lanes
      lm[i] = vmax3(m, quad_xor2(m), kLowest);
    }
    if (picking) picks(r, kslab);
    float was[NR];
    bool need[NR];
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      was[i] = mx[i];
      need[i] = !first && lm[i] > mx[i] + kSlack;
      mx[i] = (first || need[i]) ? lm[i] : mx[i];
      float e[8];
      expand(r.x[i], e);
      const float ml = mx[i] * kLog2e;
      float x[8];
#pragma unroll
      for (int j = 0; j < 8; ++j)
        x[j] = __builtin_amdgcn_exp2f(__builtin_fmaf(e[j], kLog2e, -ml));
      const Frag3 f = split8(x);
      Xs[buf][0][slot[i]] = f.h;
      Xs[buf][1][slot[i]] = f.m;
      Xs[buf][2][slot[i]] = f.l;
    }
    // rare: a row's reference moved; everything summed for it so far shrinks by exp(old - new)
    // (0 if old stood for -inf).  One uniform branch for the wavefront, after the staging.
    bool any = false;
#pragma unroll
    for (int i = 0; i < NR; ++i) any = any || need[i];
    if (__builtin_amdgcn_ballot_w64(any) != 0) {
#pragma unroll
      for (int i = 0; i < NR; ++i)
        if (need[i]) {
          if (c8 == 0) scale[srow + (kThreads / 4) * i] = __expf(was[i] - mx[i]);
          moved = 1;
        }
    }
  };

  // this wavefront's block of 32 label positions and first frame block; a label block past the
  // utterance only helps staging
  const int ublock = (u0 >> 5) + (wave & 3);
  const int mb0 = (wave >> 2) * MB;
  const bool active = 32 * ublock < Ub;
  const uint4* yw = Yp + ((size_t)b * nub + (active ? ublock : 0)) * nks * 3 * 64 + lane;
  // Y fragments of step `ks` (16 v): three coalesced 16-byte loads
  auto fetch_y = [&](int ks) -> Frag3 {
    const uint4* p = yw + (size_t)ks * 3 * 64;
    Frag3 y;
    y.h = p[0]; y.m = p[64]; y.l = p[128];
    return y;
  };

  floatx16 acc[MB], tot[MB];
#pragma unroll
  for (int m = 0; m < MB; ++m)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[m][r] = tot[m][r] = 0.0f;

  // fragment slots of this lane: row 32*(mb0 + m) + l32, v-eights 2*s + h
  int aslot[2][MB];
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int m = 0; m < MB; ++m) aslot[s][m] = xslot(32 * (mb0 + m) + l32, 2 * s + h);

  const int nk = (d.V + kSlice - 1) / kSlice;
  int cur = 0;
  // One slab: request the next slab's emissions, multiply the current one, stage the next.
  // Inside the matrix part the order is pinned with scheduling fences: the fragments of the
  // second step are read from LDS while the first step is multiplied, each piece as soon as the
  // first step's copy of it is no longer needed (so one set of fragment registers serves), and a
  // step's Y fragments are re-requested for the next slab right after their last use (one set
  // again).  Left to itself the compiler reads every fragment just before its first use and the
  // matrix instructions wait for LDS one by one.
  struct YRegs { Frag3 s0, s1; };
  auto slab = [&](int kt, YRegs& y, auto act) {
    constexpr bool kAct = decltype(act)::value;
    const int ktn = min(kt + 1, nk - 1);
    // did a row's reference move while this slab was staged?  Read together with the fragments
    // (LDS answers in order), so the flag costs no round trip of its own.
    const int mv = moved;
    const XRegs xs = fetch(ktn * kSlice);
    if (kAct) {
      uint4 ah[MB], am[MB], al[MB];
#pragma unroll
      for (int m = 0; m < MB; ++m) al[m] = Xs[cur][2][aslot[0][m]];
#pragma unroll
      for (int m = 0; m < MB; ++m) ah[m] = Xs[cur][0][aslot[0][m]];
#pragma unroll
      for (int m = 0; m < MB; ++m) am[m] = Xs[cur][1][aslot[0][m]];
      __builtin_amdgcn_sched_barrier(0);
      if (mv) {  // uniform; rare: apply the factors before the re-referenced slab is multiplied
#pragma unroll
        for (int m = 0; m < MB; ++m)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float f = scale[32 * (mb0 + m) + mfma_row(r, h)];
            acc[m][r] *= f;
            tot[m][r] *= f;
          }
      }
      // six piece products per block, smallest first; blocks interleaved so that consecutive
      // instructions do not wait on each other's accumulator
#pragma unroll
      for (int m = 0; m < MB; ++m) acc[m] = mfma_bf16(al[m], y.s0.h, acc[m]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int m = 0; m < MB; ++m) al[m] = Xs[cur][2][aslot[1][m]];
#pragma unroll
      for (int m = 0; m < MB; ++m) acc[m] = mfma_bf16(ah[m], y.s0.l, acc[m]);
#pragma unroll
      for (int m = 0; m < MB; ++m) acc[m] = mfma_bf16(am[m], y.s0.m, acc[m]);
#pragma unroll
      for (int m = 0; m < MB; ++m) acc[m] = mfma_bf16(am[m], y.s0.h, acc[m]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int m = 0; m < MB; ++m) am[m] = Xs[cur][1][aslot[1][m]];
#pragma unroll
      for (int m = 0; m < MB; ++m) acc[m] = mfma_bf16(ah[m], y.s0.m, acc[m]);
#pragma unroll
      for (int m = 0; m < MB; ++m) acc[m] = mfma_bf16(ah[m], y.s0.h, acc[m]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int m = 0; m < MB; ++m) ah[m] = Xs[cur][0][aslot[1][m]];
      y.s0 = fetch_y(2 * ktn);
#pragma unroll
      for (int m = 0; m < MB; ++m) acc[m] = mfma_bf16(al[m], y.s1.h, acc[m]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int m = 0; m < MB; ++m) acc[m] = mfma_bf16(ah[m], y.s1.l, acc[m]);
#pragma unroll
      for (int m = 0; m < MB; ++m) acc[m] = mfma_bf16(am[m], y.s1.m, acc[m]);
#pragma unroll
      for (int m = 0; m < MB; ++m) acc[m] = mfma_bf16(am[m], y.s1.h, acc[m]);
#pragma unroll
      for (int m = 0; m < MB; ++m) acc[m] = mfma_bf16(ah[m], y.s1.m, acc[m]);
#pragma unroll
      for (int m = 0; m < MB; ++m) acc[m] = mfma_bf16(ah[m], y.s1.h, acc[m]);
      __builtin_amdgcn_sched_barrier(0);
      y.s1 = fetch_y(2 * ktn + 1);
    }
    __builtin_amdgcn_sched_barrier(0);
    if (mv) {  // every wavefront has used the factors: back to 1 before the staging sets new ones
      __syncthreads();
      for (int r = tid; r < kRows; r += kThreads) scale[r] = 1.0f;
      if (tid == 0) moved = 0;
      __syncthreads();
    }
    stash(cur ^ 1, xs, false, min(kt + 1, nk - 1));
    __syncthreads();
    cur ^= 1;
  };
  __syncthreads();  // order
  next_pick();
  stash(0, fetch(0), true, 0);
  YRegs y0;
  if (active) {
    y0.s0 = fetch_y(0);
    y0.s1 = fetch_y(1);
  }
  __syncthreads();
  // Two copies of the loop, so that a wavefront with nothing to multiply is a path of its own:
  // inside one loop the counted waits for the emission loads would have to hold on both paths,
  // and the one without Y requests in flight makes the multiplying wavefronts wait for theirs.
  if (active) {
    for (int kt = 0; kt < nk; ++kt) {
      slab(kt, y0, std::true_type{});
      if ((kt + 1) % kFlush == 0) {
#pragma unroll
        for (int m = 0; m < MB; ++m)
#pragma unroll
          for (int r = 0; r < 16; ++r) { tot[m][r] += acc[m][r]; acc[m][r] = 0.0f; }
      }
    }
  } else {
    for (int kt = 0; kt < nk; ++kt) slab(kt, y0, std::false_type{});
  }

  // final references: to LDS for the write-out below, to mE for the kernels that come later
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int row = srow + (kThreads / 4) * i;
    if (c8 == 0) {
      mfin[row] = mx[i];
      if (t0 + row < d.T) mE[(size_t)b * d.T + t0 + row] = (t0 + row < Tb) ? mx[i] : 0.0f;
    }
  }
  __syncthreads();
  const int u = 32 * ublock + l32;
  if (!active) {
    // label positions past the utterance (but inside U) are written as zeros
    if (u < d.U && lnS == nullptr)
      for (int r = 0; r < 16 * MB; ++r) {
        const int t = t0 + 32 * (mb0 + (r >> 4)) + mfma_row(r & 15, h);
        if (t < d.T) LNb[(size_t)t * d.U + u] = 0.0f;
      }
    return;
  }
  const float mu = mP[(size_t)b * d.U + min(u, Ub - 1)];
#pragma unroll
  for (int m = 0; m < MB; ++m)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = 32 * (mb0 + m) + mfma_row(r, h), t = t0 + row;
      if (t < d.T && u < d.U) {
        float v = 0.0f;
        if (t < Tb && u < Ub)
          v = add3(logf(tot[m][r] + acc[m][r]), mfin[row], mu, reference_shift(mfin[row]));
        if (lnS == nullptr) LNb[(size_t)t * d.U + u] = v;
        else if (t < Tb && u < Ub) lnS[plane_at(d, b, u, t + u)] = v;
      }
    }
}

}  // namespace

template <typename TIO>
static bool lse_stream_ok(const TIO* E, const Dims& d) {
  (void)E;
  const long total = (long)((d.T + 63) / 64) * ((d.U + 127) / 128) * d.B;
  return d.V >= 1 && total < (1l << 30);
}
bool lse_stream_supported(const float* E, const Dims& d) { return lse_stream_ok(E, d); }
bool lse_stream_supported(const bf16_t* E, const Dims& d) { return lse_stream_ok(E, d); }
bool lse_stream_supported(const f16_t* E, const Dims& d) { return lse_stream_ok(E, d); }

size_t lse_scratch_bytes(const Dims& d) {
  if (d.B == 0 || d.T == 0 || d.U == 0 || d.V == 0) return 0;
  return (size_t)d.B * y_ublocks(d) * y_steps(d) * 3 * 64 * sizeof(uint4);
}

template <typename TIO>
static int yplanes_any(const TIO* P, const float* mP, void* scratch, const int* labLen,
                       const Dims& d, hipStream_t s) {
  const int nub = y_ublocks(d), nks = y_steps(d);
  const int vec4 = (reinterpret_cast<uintptr_t>(P) & 15) == 0 && d.V % RowAlign<TIO>::kElems == 0;
  hipLaunchKernelGGL(yplanes_kernel<TIO>, dim3((nks + 3) / 4, nub, d.B), dim3(256), 0, s, P, mP,
                     static_cast<uint4*>(scratch), labLen, d, nub, nks, vec4);
  RNNT_LAUNCH_CHECK("yplanes_kernel");
  return kOk;
}
int launch_yplanes(const float* P, const float* mP, void* scratch, const int* labLen,
                   const Dims& d, hipStream_t s) {
  return yplanes_any(P, mP, scratch, labLen, d, s);
}
int launch_yplanes(const bf16_t* P, const float* mP, void* scratch, const int* labLen,
                   const Dims& d, hipStream_t s) {
  return yplanes_any(P, mP, scratch, labLen, d, s);
}
int launch_yplanes(const f16_t* P, const float* mP, void* scratch, const int* labLen,
                   const Dims& d, hipStream_t s) {
  return yplanes_any(P, mP, scratch, labLen, d, s);
}

template <typename TIO>
static int lse_stream_any(const TIO* E, float* mE, const float* mP, float* LN,
                          const void* scratch, const int* inLen, const int* labLen,
                          const Dims& d, hipStream_t s, const int* labels, float* elS,
                          float* eb, float* lnS) {
  const int nub = y_ublocks(d), nks = y_steps(d);
  // Tiles of 128 frames; of 64 where those would not give every CU a workgroup (short or few
  // utterances: B=32 T=400 U=101 V=4096 is 128 tiles of 128 frames, each walking all columns on
  // a CU of its own while half the device idles).
  const int utiles = (d.U + 127) / 128;
  const bool low = (long)((d.T + 127) / 128) * utiles * d.B < 256;
  const int rows = low ? 64 : kRowsMax;
  const int ttiles = (d.T + rows - 1) / rows;
  const long total = (long)ttiles * utiles * d.B;
  const int grid = (int)((total + 7) / 8 * 8);
  constexpr int kWaves = 4;
  constexpr int kA = RowAlign<TIO>::kElems;
  const bool vec = d.V % kA == 0 && d.V >= kA && (reinterpret_cast<uintptr_t>(E) & 15) == 0;
#define RNNT_LSE_LAUNCH(VEC, ROWS)                                                            \
  hipLaunchKernelGGL((lse_stream_kernel<kWaves, TIO, VEC, ROWS>), dim3(grid),                 \
                     dim3(64 * kWaves), 0, s, E, mE, mP, static_cast<const uint4*>(scratch),  \
                     LN, inLen, labLen, d, ttiles, utiles, (int)total, nub, nks, labels, elS, \
                     eb, lnS)
  if (vec && low) RNNT_LSE_LAUNCH(true, 64);
  else if (vec) RNNT_LSE_LAUNCH(true, kRowsMax);
  else if (low) RNNT_LSE_LAUNCH(false, 64);
  else RNNT_LSE_LAUNCH(false, kRowsMax);
#undef RNNT_LSE_LAUNCH
  RNNT_LAUNCH_CHECK("lse_stream_kernel");
  return kOk;
}
int launch_lse_stream(const float* E, float* mE, const float* mP, float* LN,
                      const void* scratch, const int* inLen, const int* labLen, const Dims& d,
                      hipStream_t s, const int* labels, float* elS, float* eb,
                      float* lnS) {
  return lse_stream_any(E, mE, mP, LN, scratch, inLen, labLen, d, s, labels, elS, eb, lnS);
}
int launch_lse_stream(const bf16_t* E, float* mE, const float* mP, float* LN,
                      const void* scratch, const int* inLen, const int* labLen, const Dims& d,
                      hipStream_t s, const int* labels, float* elS, float* eb,
                      float* lnS) {
  return lse_stream_any(E, mE, mP, LN, scratch, inLen, labLen, d, s, labels, elS, eb, lnS);
}
int launch_lse_stream(const f16_t* E, float* mE, const float* mP, float* LN,
                      const void* scratch, const int* inLen, const int* labLen, const Dims& d,
                      hipStream_t s, const int* labels, float* elS, float* eb,
                      float* lnS) {
  return lse_stream_any(E, mE, mP, LN, scratch, inLen, labLen, d, s, labels, elS, eb, lnS);
}

}  // namespace rnnt
