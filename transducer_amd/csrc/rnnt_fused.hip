// Both dense gradients of the loss (transducer/torch_binding.py:85-89) from ONE walk over the
// frames, for gfx950:
//
//   egrads[t,v] = delta * X[t,v] * sum_u W[t,u] * Y[u,v]      X = exp(E - mE), Y = exp(P - mP)
//   pgrads[u,v] = delta * Y[u,v] * sum_t W[t,u] * X[t,v]
//
// The two separate contractions (rnnt_grads.hip) give a wavefront the same unit of work -- 32
// columns v of one utterance, all of its frames, 32 at a time -- and each reads the slab of E
// and forms X from it.  Here one wavefront does both: the slab is read once and turned into X
// once; X scales the finished egrads block on its way out (lane = column, registers = the
// block's frames) and, split into its three bf16 pieces, is the B operand of the pgrads
// products.  The matrix instruction sums over its k axis in any order as long as both operands
// agree on it, so the frames of a slab are fed to the pgrads products in the order the egrads
// block holds them, and the W^T slab comes in that same order (WImages): X never moves
// between lanes.
//
// One wavefront per SIMD with the whole register file: the Y pieces (84 registers), the pgrads
// sums (64) and the egrads block (32) live in the accumulation registers, where the matrix
// instructions read and write them directly; the vector registers hold X, its pieces, the next
// slab's emissions (requested a slab ahead: there is no second wavefront to cover the wait)
// and the staging of the next W slabs.  W arrives already split into pieces (post_beta_kernel
// writes the slab images), so staging is a plain 16-byte copy: with a lone wavefront the issue
// slots of the vector ALU are what is scarce.  The matrix instructions are written as inline
// assembly, because that is the only way to pin their operands to the accumulation registers;
// the hazards the compiler would otherwise guard are handled here (see mfma_* below).
//
// Same products as the two separate kernels: six piece products per 32x32x16 block, smallest
// first.  egrads comes out with the same bits; pgrads sums its frames in one level (see pacc).
#include <type_traits>

#include "rnnt_internal.h"
#include "rnnt_io.h"
#include "rnnt_split.h"
#include "rnnt_grads.h"

namespace rnnt {

namespace {

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

// acc (accumulation registers) += A (vector registers) x B.  The accumulators are only ever
// touched by these instructions, by the guarded reads below and by the compiler's own
// v_accvgpr moves; back-to-back instructions on one accumulator are interlocked by the hardware.
__device__ __forceinline__ void mfma_acc_ab(floatx16& acc, u32x4 a, u32x4 b_acc) {
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "a"(b_acc));
}
__device__ __forceinline__ void mfma_acc_vv(floatx16& acc, u32x4 a, u32x4 b) {
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc) : "v"(a), "v"(b));
}
// the first product of a sum: acc = A x B + 0 (no clearing of the accumulator beforehand)
__device__ __forceinline__ void mfma_new_ab(floatx16& acc, u32x4 a, u32x4 b_acc) {
  asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&a"(acc) : "v"(a), "a"(b_acc));
}
// Before the vector ALU reads an accumulator a matrix instruction wrote: that instruction needs
// 18 cycles after issue (the compiler inserts them for its own instructions; it does not know
// what the assembly above is).
__device__ __forceinline__ void mfma_settle(floatx16& a) {
  asm volatile("s_nop 15\n\ts_nop 3" : "+a"(a));
}
__device__ __forceinline__ void mfma_settle(floatx16& a, floatx16& b) {
  asm volatile("s_nop 15\n\ts_nop 3" : "+a"(a), "+a"(b));
}
// After the vector ALU wrote an accumulator (v_accvgpr_write) and before a matrix instruction
// reads it.
__device__ __forceinline__ void mfma_after_write(floatx16& a) {
  asm volatile("s_nop 7" : "+a"(a));
}
__device__ __forceinline__ u32x4 to_acc(const uint4& v) {
  u32x4 r = {v.x, v.y, v.z, v.w};
  asm volatile("" : "+a"(r));  // lives in the accumulation registers from here on
  return r;
}
__device__ __forceinline__ u32x4 vec(const uint4& v) { return u32x4{v.x, v.y, v.z, v.w}; }
// A 32-bit byte offset that the compiler must take as it is, inside the loop: added to a
// uniform base it then becomes the scalar-base + 32-bit-offset form of a global access (one
// register, no address arithmetic).  Left alone, the compiler widens the loop-invariant
// offsets to 64 bits ahead of the loop and spends two registers and a 64-bit add per access.
__device__ __forceinline__ unsigned as_is(unsigned x) {
  asm volatile("" : "+v"(x));
  return x;
}

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): a loop whose index is a
// compile-time constant inside the body (which register, which accumulator, which unit of work
// rides behind which matrix instruction: all decided at compile time).
template <int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (N > 0) {
    static_for<N - 1>(f);
    f(std::integral_constant<int, N - 1>());
  }
}

// LDS image of the two W slabs of one frame tile (double-buffered by the kernel).  Rows are
// padded so that the 16-byte fragment reads of 8 consecutive rows fall into distinct bank
// groups (kEsPitch, kPsPitch).
struct FusedLds {
  unsigned short Ae[2][3][kEsPlane];     // frames x label positions (egrads' A operand)
  unsigned short Ap[2][3][kPsPlane];     // label positions x frame slots (pgrads' A operand)
  float Ms[2][32];                       // mE * log2(e) of the slab's frames
  float Strip[4][32];                    // per wavefront: sparse terms of egrads
  unsigned short Match[4][kMaxLabels];   // per wavefront: label positions whose label is one of
                                         // its 32 columns
  PRowTerms Rt;
};

template <int NS, int NMB, typename TIO>
__device__ __forceinline__ void fused_walk(
    const TIO* __restrict__ E, const TIO* __restrict__ P, const float* __restrict__ mE,
    const float* __restrict__ mP, const WImages& img, const float* __restrict__ deltas,
    TIO* __restrict__ egrads, TIO* __restrict__ pgrads, FusedLds& L, const Dims& d, int Tw,
    int b, int Tb, int Ub, const SparseTerms& sp, int nmatch) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, h = lane >> 5;
  const int wave_col0 = blockIdx.x * 128 + wave * 32;
  const int vcol = wave_col0 + l32;
  const bool vok = vcol < d.V;
  const int vc = vok ? vcol : d.V - 1;
  const bool cols_full = wave_col0 + 32 <= d.V;
  const unsigned short* match = L.Match[wave];
  const int blank_lane =
      (d.blank >= wave_col0 && d.blank < wave_col0 + 32) ? d.blank - wave_col0 : -1;
  const int ntiles = (d.T + 31) >> 5;
  const int tile_valid = (Tb + 31) >> 5;  // >= 1: utterances without frames never get here
  const float delta = deltas ? deltas[b] : 1.0f;
  const TIO* Eb = E + (size_t)b * d.T * d.V;
  TIO* eout = egrads + (size_t)b * d.T * d.V;
  const float* mEb = mE + (size_t)b * d.T;
  const TIO* Pb = P + (size_t)b * d.U * d.V;
  const float* mPb = mP + (size_t)b * d.U;

  // byte offset, inside a frame tile of E (and of egrads: same layout), of the element that
  // register r of this lane holds: frame mfma_row(r, h), column vc
  unsigned off[16];
#pragma unroll
  for (int r = 0; r < 16; ++r)
    off[r] = ((unsigned)mfma_row(r, h) * (unsigned)d.V + (unsigned)vc) * (unsigned)sizeof(TIO);
  // full: the tile lies wholly inside the utterance (known to the caller: the loop over full
  // tiles must not have a branch here, see `tile` below)
  auto load_e = [&](int ti, float (&e)[16], auto full) __attribute__((always_inline)) {
    const int t0 = ti * 32;
    const char* base = reinterpret_cast<const char*>(Eb + (size_t)t0 * d.V);
    if constexpr (decltype(full)::value) {
#pragma unroll
      for (int r = 0; r < 16; ++r) e[r] = ldf(reinterpret_cast<const TIO*>(base + as_is(off[r])));
    } else {
      // rows past the utterance are read from its last frame: masked on the way out of egrads,
      // multiplied by the zeros of W^T in pgrads
#pragma unroll
      for (int r = 0; r < 16; ++r)
        e[r] = ldf(Eb + (size_t)min(t0 + mfma_row(r, h), Tb - 1) * d.V + vc);
    }
  };

  // The first tile's emissions are requested before everything else: the wait the compiler
  // places ahead of their first use in the loop below must hold for the loop's first trip too,
  // and it names how many requests may still be out -- with these issued last before the loop
  // it would make EVERY trip wait for the requests it has just issued (the next slabs and the
  // next tile's emissions).
  // (three register sets: a fast tile requests the emissions of the tile after the next one --
  // with one wavefront per SIMD only 4 KB per wavefront are in flight per tile requested, and a
  // request made one tile ahead comes back too late once a tile takes less than the memory
  // latency under load)
  float evA[16], evB[16], evC[16];
  load_e(0, evA, std::false_type());
  load_e(min(1, tile_valid - 1), evB, std::false_type());

  // Y fragments (egrads' B operand), in the accumulation registers: step s holds label
  // positions 16 s + 8 h + i
  u32x4 yh[NS], ym[NS], yl[NS];
  {
    float praw[NS][8], mraw[NS][8];
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int u = 16 * s + 8 * h + i;
        const int uc = u < Ub ? u : 0;
        praw[s][i] = ldf(Pb + (size_t)uc * d.V + vc);
        mraw[s][i] = mPb[uc];
      }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      float y[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int u = 16 * s + 8 * h + i;
        const float e = __expf(praw[s][i] - mraw[s][i]);
        y[i] = (u < Ub && vok) ? e : 0.0f;
      }
      const Frag3 f = split8(y);
      yh[s] = to_acc(f.h);
      ym[s] = to_acc(f.m);
      yl[s] = to_acc(f.l);
    }
  }

  // Staging of a frame tile's two W slab images: 16-byte chunks, copied as they are.  Of the
  // egrads image the first 2 NS chunks of each row, of the pgrads image the first 32 NMB rows.
  constexpr int kEChunks = 3 * 32 * 2 * NS, kPChunks = 3 * 32 * NMB * 4;
  constexpr int kNE = (kEChunks + 255) / 256, kNP = (kPChunks + 255) / 256;
  unsigned e_src[kNE], e_dst[kNE], p_src[kNP], p_dst[kNP];  // byte offsets
#pragma unroll
  for (int i = 0; i < kNE; ++i) {
    const int c = min(tid + 256 * i, kEChunks - 1);  // (a thread past the end repeats the last)
    const int plane = c / (64 * NS), rem = c - plane * (64 * NS);
    const int row = rem / (2 * NS), j = rem - row * (2 * NS);
    e_src[i] = (unsigned)(plane * WImages::kEPlane * 4 + row * (WImages::kCols * 2) + j * 16);
    e_dst[i] = (unsigned)(plane * kEsPlane * 2 + row * kEsPitch * 2 + j * 16);
  }
#pragma unroll
  for (int i = 0; i < kNP; ++i) {
    const int c = min(tid + 256 * i, kPChunks - 1);
    const int plane = c / (128 * NMB), rem = c - plane * (128 * NMB);
    const int row = rem >> 2, j = rem & 3;
    p_src[i] = (unsigned)(plane * WImages::kPPlane * 4 + row * 64 + j * 16);
    p_dst[i] = (unsigned)(plane * kPsPlane * 2 + row * kPsPitch * 2 + j * 16);
  }
  const size_t img_tile0 = (size_t)b * (Tw >> 5);
  struct Staged {
    u32x4 e[kNE], p[kNP];
    float m;
  };
  auto fetch = [&](int ti) -> Staged {
    Staged s;
    const char* es = reinterpret_cast<const char*>(img.e + (img_tile0 + ti) * (3 * WImages::kEPlane));
    const char* ps = reinterpret_cast<const char*>(img.p + (img_tile0 + ti) * (3 * WImages::kPPlane));
#pragma unroll
    for (int i = 0; i < kNE; ++i) s.e[i] = *reinterpret_cast<const u32x4*>(es + as_is(e_src[i]));
#pragma unroll
    for (int i = 0; i < kNP; ++i) s.p[i] = *reinterpret_cast<const u32x4*>(ps + as_is(p_src[i]));
    s.m = mEb[min(ti * 32 + (tid & 31), Tb - 1)];
    return s;
  };
  auto stage = [&](int buf, const Staged& s) {
    char* ed = reinterpret_cast<char*>(&L.Ae[buf][0][0]);
    char* pd = reinterpret_cast<char*>(&L.Ap[buf][0][0]);
#pragma unroll
    for (int i = 0; i < kNE; ++i) *reinterpret_cast<u32x4*>(ed + e_dst[i]) = s.e[i];
#pragma unroll
    for (int i = 0; i < kNP; ++i) *reinterpret_cast<u32x4*>(pd + p_dst[i]) = s.p[i];
    if (tid < 32) L.Ms[buf][tid] = s.m * kLog2e;
  };

  // the first kEsPrefetch matches of the folded label terms, resolved once
  int mu[kEsPrefetch], mc[kEsPrefetch];
#pragma unroll
  for (int i = 0; i < kEsPrefetch; ++i) {
    mu[i] = i < nmatch ? match[i] : 0;
    mc[i] = i < nmatch ? label_at(sp.labels, d, b, mu[i]) - wave_col0 : -1;
  }

  // pgrads' sums over the frames, one level (the separate kernel moves its running sums into a
  // second level every kPsFlush slabs, because the matrix instruction truncates what falls
  // below the accumulator's last bit and a long sum drifts low: 2e-6 relative over 2000 frames,
  // a fiftieth of the gradients' tolerance; here the 64 registers of a second level are what
  // decides between a loop without spills and one with)
  floatx16 pacc[NMB];
#pragma unroll
  for (int mb = 0; mb < NMB; ++mb) {
#pragma unroll
    for (int r = 0; r < 16; ++r) pacc[mb][r] = 0.0f;
    mfma_after_write(pacc[mb]);
  }

  int cur = 0;
  stage(0, fetch(0));
  __syncthreads();

  // One frame tile, general form (the utterance's last tiles, the last column block, wavefronts
  // with more folded labels than the fast form prefetches): `evc` holds its emissions, `evn`
  // receives the next tile's.
  auto tile = [&](int ti, float (&evc)[16], float (&evn)[16]) __attribute__((always_inline)) {
    const std::false_type full;
    const bool interior = cols_full && (ti * 32 + 32 <= Tb);
    const int t0 = ti * 32;
    const int tnext = min(ti + 1, tile_valid - 1);
    // Requests in the order their answers are needed (they come back in order, and a wait
    // names how many requests may still be out): this tile's blank / label terms, the next
    // tile's W slabs (stored to LDS at the end of this tile), the next tile's emissions (not
    // needed before the next tile).
    float sd[kEsPrefetch], sbl = 0.0f;
    if (nmatch > 0 || blank_lane >= 0) {
      const int tr = min(t0 + l32, Tb - 1);
#pragma unroll
      for (int i = 0; i < kEsPrefetch; ++i) {
        sd[i] = sp.emT[((size_t)b * d.U + mu[i]) * d.T + tr];
      }
      if (blank_lane >= 0) sbl = sp.bsum[(size_t)b * d.T + tr];
    }
    asm volatile("" ::: "memory");  // (the compiler must not reorder the three groups)
    const Staged nxt = fetch(tnext);  // (the last tile re-reads its own: no branch around loads)
    asm volatile("" ::: "memory");
    load_e(tnext, evn, full);  // (a full tile of the loop is followed by a full one)
    asm volatile("" ::: "memory");
    const char* ae = reinterpret_cast<const char*>(&L.Ae[cur][0][0]) + l32 * kEsPitch * 2 + 16 * h;
    const char* ap = reinterpret_cast<const char*>(&L.Ap[cur][0][0]) + l32 * kPsPitch * 2 + 16 * h;
    auto e_frag = [&](int plane, int s) {
      return *reinterpret_cast<const u32x4*>(ae + plane * kEsPlane * 2 + 32 * s);
    };
    auto p_frag = [&](int plane, int mb, int s) {
      return *reinterpret_cast<const u32x4*>(ap + plane * kPsPlane * 2 + mb * 32 * kPsPitch * 2 + 32 * s);
    };
    // LDS reads are issued in program order and are not moved across the matrix instructions
    // (inline assembly), so what follows is software-pipelined by hand: every fragment is
    // requested one group of matrix instructions before the group that uses it.
    u32x4 eh = e_frag(0, 0), em = e_frag(1, 0), el = e_frag(2, 0);
    // X of this tile: register r = frame mfma_row(r, h) of column l32
    float x[16];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const float4 m4 = *reinterpret_cast<const float4*>(&L.Ms[cur][8 * g + 4 * h]);
#pragma unroll
      for (int k = 0; k < 4; ++k) x[4 * g + k] = exp_minus_scaled(evc[4 * g + k], f4at(m4, k));
    }
    // pgrads takes its label blocks two at a time (alternating accumulators); the groups of a
    // tile: (k-step 0 | 1) x (blocks 0,1 | blocks 2,3)
    constexpr int kPairs = (NMB + 1) / 2, kGroups = 2 * kPairs;
    struct PFrags { u32x4 h[2], m[2], l[2]; };
    auto p_group = [&](int g) -> PFrags {
      const int s = g / kPairs, mb0 = 2 * (g % kPairs);
      PFrags f;
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        const int mb = mb0 + k < NMB ? mb0 + k : mb0;  // (an odd block count: the last one alone)
        f.h[k] = p_frag(0, mb, s);
        f.m[k] = p_frag(1, mb, s);
        f.l[k] = p_frag(2, mb, s);
      }
      return f;
    };
    // egrads: W slab (rows = frames) x Y, two accumulators.  The pieces of X (pgrads' B operand)
    // are formed between the steps, where the vector ALU has nothing else to do.
    floatx16 acc, acc2;
    u32x4 xh[2], xm[2], xl[2];
    PFrags pf;
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      const u32x4 ch = eh, cm = em, cl = el;
      if (s + 1 < NS) {
        eh = e_frag(0, s + 1);
        em = e_frag(1, s + 1);
        el = e_frag(2, s + 1);
      } else {
        pf = p_group(0);
      }
      if (s == 0) {
        mfma_new_ab(acc, cl, yh[0]);
        mfma_new_ab(acc2, ch, yl[0]);
      } else {
        mfma_acc_ab(acc, cl, yh[s]);
        mfma_acc_ab(acc2, ch, yl[s]);
      }
      mfma_acc_ab(acc, cm, ym[s]);
      mfma_acc_ab(acc2, cm, yh[s]);
      mfma_acc_ab(acc, ch, ym[s]);
      mfma_acc_ab(acc2, ch, yh[s]);
      if (s < 2) {
        float xs[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) xs[i] = x[8 * s + i];
        const Frag3 xf = split8(xs);
        xh[s] = vec(xf.h);
        xm[s] = vec(xf.m);
        xl[s] = vec(xf.l);
      }
    }
    // pgrads: W^T slab (rows = label positions) x X; the pieces of X for k-step s are those of
    // registers 8 s .. 8 s + 7
#pragma unroll
    for (int g = 0; g < kGroups; ++g) {
      const PFrags c = pf;
      if (g + 1 < kGroups) pf = p_group(g + 1);
      const int s = g / kPairs, mb0 = 2 * (g % kPairs);
      if (mb0 + 1 < NMB) {
        floatx16& p0 = pacc[mb0];
        floatx16& p1 = pacc[mb0 + 1 < NMB ? mb0 + 1 : mb0];
        mfma_acc_vv(p0, c.l[0], xh[s]);
        mfma_acc_vv(p1, c.l[1], xh[s]);
        mfma_acc_vv(p0, c.h[0], xl[s]);
        mfma_acc_vv(p1, c.h[1], xl[s]);
        mfma_acc_vv(p0, c.m[0], xm[s]);
        mfma_acc_vv(p1, c.m[1], xm[s]);
        mfma_acc_vv(p0, c.m[0], xh[s]);
        mfma_acc_vv(p1, c.m[1], xh[s]);
        mfma_acc_vv(p0, c.h[0], xm[s]);
        mfma_acc_vv(p1, c.h[1], xm[s]);
        mfma_acc_vv(p0, c.h[0], xh[s]);
        mfma_acc_vv(p1, c.h[1], xh[s]);
      } else {
        floatx16& p0 = pacc[mb0];
        mfma_acc_vv(p0, c.l[0], xh[s]);
        mfma_acc_vv(p0, c.h[0], xl[s]);
        mfma_acc_vv(p0, c.m[0], xm[s]);
        mfma_acc_vv(p0, c.m[0], xh[s]);
        mfma_acc_vv(p0, c.h[0], xm[s]);
        mfma_acc_vv(p0, c.h[0], xh[s]);
      }
    }
    // the next tile's W slabs into the other LDS buffer (free since the last barrier); ahead of
    // the stores below, so that its wait only has the next tile's emissions behind it
    stage(cur ^ 1, nxt);
    // egrads write-out
    mfma_settle(acc, acc2);
    float v[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const float y = x[r] * (acc[r] + acc2[r]);
      v[r] = (interior || t0 + mfma_row(r, h) < Tb) ? y : 0.0f;
    }
    if (nmatch > 0 || blank_lane >= 0) {  // uniform per wavefront, and rare
      const bool row_ok = t0 + l32 < Tb;
      float* strip = &L.Strip[wave][0];
      auto apply = [&](float term, int col, float sign) {
        if (h == 0) strip[l32] = term;
        if (l32 == col) {
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const float4 q = *reinterpret_cast<const float4*>(&strip[8 * g + 4 * h]);
            v[4 * g + 0] += sign * q.x;
            v[4 * g + 1] += sign * q.y;
            v[4 * g + 2] += sign * q.z;
            v[4 * g + 3] += sign * q.w;
          }
        }
      };
#pragma unroll
      for (int i = 0; i < kEsPrefetch; ++i)
        if (i < nmatch) apply(row_ok ? sd[i] : 0.0f, mc[i], -1.0f);
      for (int i = kEsPrefetch; i < nmatch; ++i) {
        const int u = match[i];
        apply(row_ok ? sp.emT[((size_t)b * d.U + u) * d.T + min(t0 + l32, Tb - 1)] : 0.0f,
              label_at(sp.labels, d, b, u) - wave_col0, -1.0f);
      }
      if (blank_lane >= 0) apply(row_ok ? sbl : 0.0f, blank_lane, 1.0f);
    }
    if (interior) {
      char* obase = reinterpret_cast<char*>(eout + (size_t)t0 * d.V);
#pragma unroll
      for (int r = 0; r < 16; ++r) stf(reinterpret_cast<TIO*>(obase + as_is(off[r])), delta * v[r]);
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int t = t0 + mfma_row(r, h);
        if (t < d.T && vok) stf(eout + (size_t)t * d.V + vcol, delta * v[r]);
      }
    }
    __syncthreads();
    cur ^= 1;
  };
  // The same tile for the common case -- all 32 frames inside the utterance (and the next tile's
  // too), all 32 columns inside the vocabulary, at most kEsPrefetch folded labels -- scheduled by
  // hand.  A lone wavefront issues in order: a matrix instruction occupies its pipe for 32
  // cycles, and the five or six other instructions that can issue meanwhile must stand right
  // behind it in the instruction stream.  So everything else a tile has to do is cut into small
  // units and dealt out between the matrix instructions, with scheduling barriers that keep
  // the compiler from regrouping them:
  //   egrads products (6 NS): the next tile's requests (W slabs first, then emissions: waits
  //     count requests in order), this tile's X (exponentials) and its pieces, the fragment
  //     reads of the next step;
  //   pgrads products: the fragment reads of the next group, the egrads write-out row by row,
  //     the copy of the next W slabs into the other LDS buffer.
  // No branch anywhere (see the remark on waits at load_e).
  // `foldc`: the blank / label terms of this lane's sixteen frames of the tile (zero for all but
  // the one or two lanes whose column is a label's or the blank's), replaced by the next tile's
  // at the end.  They are requested at the top of a tile and exchanged through LDS at its end, the
  // only two places of the tile with a branch (a branch in the middle would cut the tile into
  // basic blocks, and the compiler moves arithmetic into the block that uses its result).
  const bool folding = nmatch > 0 || blank_lane >= 0;  // uniform per wavefront
  struct FoldRaw { float sd[kEsPrefetch], sbl; };
  auto fold_request = [&](int ti) -> FoldRaw {
    FoldRaw f;
#pragma unroll
    for (int i = 0; i < kEsPrefetch; ++i) f.sd[i] = 0.0f;
    f.sbl = 0.0f;
    if (folding) {
      const int tr = ti * 32 + l32;
#pragma unroll
      for (int i = 0; i < kEsPrefetch; ++i) {
        f.sd[i] = sp.emT[((size_t)b * d.U + mu[i]) * d.T + tr];
      }
      if (blank_lane >= 0) f.sbl = sp.bsum[(size_t)b * d.T + tr];
    }
    return f;
  };
  auto fold_exchange = [&](const FoldRaw& f, float (&fold)[16]) __attribute__((always_inline)) {
    if (folding) {
#pragma unroll
      for (int r = 0; r < 16; ++r) fold[r] = 0.0f;
      float* strip = &L.Strip[wave][0];
      auto take = [&](float term, int col, float sign) {
        if (h == 0) strip[l32] = term;
        if (l32 == col) {
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const float4 q = *reinterpret_cast<const float4*>(&strip[8 * g + 4 * h]);
            fold[4 * g + 0] += sign * q.x;
            fold[4 * g + 1] += sign * q.y;
            fold[4 * g + 2] += sign * q.z;
            fold[4 * g + 3] += sign * q.w;
          }
        }
      };
#pragma unroll
      for (int i = 0; i < kEsPrefetch; ++i)
        if (i < nmatch) take(f.sd[i], mc[i], -1.0f);
      if (blank_lane >= 0) take(f.sbl, blank_lane, 1.0f);
    }
  };
  auto fast_tile = [&](int ti, float (&evc)[16], float (&evn)[16], float (&foldc)[16])
                       __attribute__((always_inline)) {
    const int t0 = ti * 32, tnext = ti + 1;  // W slabs: the next tile's; emissions: the one after
    const FoldRaw fraw = fold_request(tnext);
    const char* ae = reinterpret_cast<const char*>(&L.Ae[cur][0][0]) + l32 * kEsPitch * 2 + 16 * h;
    const char* ap = reinterpret_cast<const char*>(&L.Ap[cur][0][0]) + l32 * kPsPitch * 2 + 16 * h;
    auto e_frag = [&](int plane, int s) {
      return *reinterpret_cast<const u32x4*>(ae + plane * kEsPlane * 2 + 32 * s);
    };
    auto p_frag = [&](int plane, int mb, int s) {
      return *reinterpret_cast<const u32x4*>(ap + plane * kPsPlane * 2 + mb * 32 * kPsPitch * 2 + 32 * s);
    };
    constexpr int kPairs = (NMB + 1) / 2, kGroups = 2 * kPairs;
    struct PFrags { u32x4 h[2], m[2], l[2]; };
    auto p_group = [&](int g) -> PFrags {
      const int s = g / kPairs, mb0 = 2 * (g % kPairs);
      PFrags f;
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        const int mb = mb0 + k < NMB ? mb0 + k : mb0;
        f.h[k] = p_frag(0, mb, s);
        f.m[k] = p_frag(1, mb, s);
        f.l[k] = p_frag(2, mb, s);
      }
      return f;
    };
    u32x4 eh = e_frag(0, 0), em = e_frag(1, 0), el = e_frag(2, 0);
    float4 m4[4];
#pragma unroll
    for (int g = 0; g < 4; ++g) m4[g] = *reinterpret_cast<const float4*>(&L.Ms[cur][8 * g + 4 * h]);
    // the next tile's requests, one at a time: W slabs (egrads image, pgrads image, the frames'
    // references), then the emissions
    Staged nxt;
    const char* es = reinterpret_cast<const char*>(img.e + (img_tile0 + tnext) * (3 * WImages::kEPlane));
    const char* ps = reinterpret_cast<const char*>(img.p + (img_tile0 + tnext) * (3 * WImages::kPPlane));
    const char* eb = reinterpret_cast<const char*>(Eb + (size_t)(ti + 2) * 32 * d.V);
    constexpr int kReq = kNE + kNP + 1 + 16;
    auto request = [&](auto icc) __attribute__((always_inline)) {
      constexpr int i = decltype(icc)::value;
      if constexpr (i < kNE) nxt.e[i] = *reinterpret_cast<const u32x4*>(es + as_is(e_src[i]));
      else if constexpr (i < kNE + kNP) nxt.p[i - kNE] = *reinterpret_cast<const u32x4*>(ps + as_is(p_src[i - kNE]));
      else if constexpr (i == kNE + kNP) nxt.m = mEb[tnext * 32 + (tid & 31)];
      else evn[i - kNE - kNP - 1] = ldf(reinterpret_cast<const TIO*>(eb + as_is(off[i - kNE - kNP - 1])));
    };
    // this tile's X and its pieces, in twelve units: four exponentials each (0..3), then the
    // pieces of two neighbouring registers each (4..11)
    float x[16];
    unsigned xph[8], xpm[8], xpl[8];
    auto x_unit = [&](auto jcc) __attribute__((always_inline)) {
      constexpr int j = decltype(jcc)::value;
      // (the empty statements tie a unit's arithmetic to this point of the instruction stream:
      // pure arithmetic has no place of its own and the compiler would gather it elsewhere)
      if constexpr (j < 4) {
        asm volatile("" : "+v"(m4[j].x), "+v"(m4[j].y), "+v"(m4[j].z), "+v"(m4[j].w));
#pragma unroll
        for (int k = 0; k < 4; ++k) x[4 * j + k] = exp_minus_scaled(evc[4 * j + k], f4at(m4[j], k));
      } else {
        constexpr int q = j - 4;
        asm volatile("" : "+v"(x[2 * q]), "+v"(x[2 * q + 1]));
        split_pair(x[2 * q], x[2 * q + 1], xph[q], xpm[q], xpl[q]);
      }
    };
    // ---- egrads products
    floatx16 acc, acc2;
    PFrags pf;
    u32x4 ch, cm, cl;
    constexpr int kProdE = 6 * NS;
    static_for<kProdE>([&](auto ic) __attribute__((always_inline)) {
      constexpr int m = decltype(ic)::value, s = m / 6, pr = m % 6;
      if constexpr (pr == 0) {
        ch = eh; cm = em; cl = el;
        if constexpr (s + 1 < NS) {
          eh = e_frag(0, s + 1);
          em = e_frag(1, s + 1);
          el = e_frag(2, s + 1);
        } else {
          pf = p_group(0);
        }
      }
      if constexpr (m == 0) mfma_new_ab(acc, cl, yh[0]);
      else if constexpr (m == 1) mfma_new_ab(acc2, ch, yl[0]);
      else if constexpr (pr == 0) mfma_acc_ab(acc, cl, yh[s]);
      else if constexpr (pr == 1) mfma_acc_ab(acc2, ch, yl[s]);
      else if constexpr (pr == 2) mfma_acc_ab(acc, cm, ym[s]);
      else if constexpr (pr == 3) mfma_acc_ab(acc2, cm, yh[s]);
      else if constexpr (pr == 4) mfma_acc_ab(acc, ch, ym[s]);
      else mfma_acc_ab(acc2, ch, yh[s]);
      // what rides behind this product
      constexpr int r0 = m * kReq / kProdE, r1 = (m + 1) * kReq / kProdE;
      static_for<r1 - r0>([&](auto jc) __attribute__((always_inline)) {
        request(std::integral_constant<int, r0 + decltype(jc)::value>());
      });
      constexpr int x0 = m * 12 / kProdE, x1 = (m + 1) * 12 / kProdE;
      static_for<x1 - x0>([&](auto jc) __attribute__((always_inline)) {
        x_unit(std::integral_constant<int, x0 + decltype(jc)::value>());
      });
      __builtin_amdgcn_sched_barrier(0);
    });
    u32x4 xh[2], xm[2], xl[2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      xh[s] = u32x4{xph[4 * s], xph[4 * s + 1], xph[4 * s + 2], xph[4 * s + 3]};
      xm[s] = u32x4{xpm[4 * s], xpm[4 * s + 1], xpm[4 * s + 2], xpm[4 * s + 3]};
      xl[s] = u32x4{xpl[4 * s], xpl[4 * s + 1], xpl[4 * s + 2], xpl[4 * s + 3]};
    }

    // ---- pgrads products; behind them the egrads write-out (16 rows), then the copy of the
    // next W slabs into the other LDS buffer (free since the last barrier)
    char* obase = reinterpret_cast<char*>(eout + (size_t)t0 * d.V);
    char* ed = reinterpret_cast<char*>(&L.Ae[cur ^ 1][0][0]);
    char* pd = reinterpret_cast<char*>(&L.Ap[cur ^ 1][0][0]);
    constexpr int kUnits = 16 + kNE + kNP + 1;
    auto p_unit = [&](auto jc) __attribute__((always_inline)) {
      constexpr int j = decltype(jc)::value;
      if constexpr (j < 16) {
        const float y = x[j] * (acc[j] + acc2[j]) + foldc[j];
        stf(reinterpret_cast<TIO*>(obase + as_is(off[j])), delta * y);
      } else if constexpr (j < 16 + kNE) {
        *reinterpret_cast<u32x4*>(ed + e_dst[j - 16]) = nxt.e[j - 16];
      } else if constexpr (j < 16 + kNE + kNP) {
        *reinterpret_cast<u32x4*>(pd + p_dst[j - 16 - kNE]) = nxt.p[j - 16 - kNE];
      } else {
        if (tid < 32) L.Ms[cur ^ 1][tid] = nxt.m * kLog2e;
      }
    };
    constexpr int kProdP = 6 * NMB * 2;  // 6 products x NMB blocks x 2 k-steps
    static_for<kGroups>([&](auto gc) __attribute__((always_inline)) {
      constexpr int g = decltype(gc)::value, s = g / kPairs, mb0 = 2 * (g % kPairs);
      constexpr bool two = mb0 + 1 < NMB;
      constexpr int n = two ? 12 : 6;
      constexpr int before = s * 6 * NMB + 12 * (g % kPairs);  // products issued before this group
      const PFrags c = pf;
      static_for<n>([&](auto kc) __attribute__((always_inline)) {
        constexpr int k = decltype(kc)::value;
        constexpr int pr = two ? k / 2 : k, w = two ? k % 2 : 0;
        constexpr int done = before + k;
        floatx16& pa = pacc[mb0 + w];
        if constexpr (pr == 0) mfma_acc_vv(pa, c.l[w], xh[s]);
        else if constexpr (pr == 1) mfma_acc_vv(pa, c.h[w], xl[s]);
        else if constexpr (pr == 2) mfma_acc_vv(pa, c.m[w], xm[s]);
        else if constexpr (pr == 3) mfma_acc_vv(pa, c.m[w], xh[s]);
        else if constexpr (pr == 4) mfma_acc_vv(pa, c.h[w], xm[s]);
        else mfma_acc_vv(pa, c.h[w], xh[s]);
        if constexpr (k == 0 && g + 1 < kGroups) pf = p_group(g + 1);
        // (the write-out reads the egrads sums: not before they have settled, two products
        // after the last egrads one)
        if constexpr (done == 1) mfma_settle(acc, acc2);
        if constexpr (done >= 2) {
          constexpr int j0 = (done - 2) * kUnits / (kProdP - 2), j1 = (done - 1) * kUnits / (kProdP - 2);
          static_for<j1 - j0>([&](auto jc) __attribute__((always_inline)) {
            p_unit(std::integral_constant<int, j0 + decltype(jc)::value>());
          });
        }
        __builtin_amdgcn_sched_barrier(0);
      });
    });
    fold_exchange(fraw, foldc);  // (this tile's terms are used up: the next tile's in their place)
    __syncthreads();
    cur ^= 1;
  };

  // full tiles first, two per trip (the two register sets of the emissions swap roles); the
  // tile after a pair must be full as well, since the pair requests its emissions
  const int tile_full = (cols_full && nmatch <= kEsPrefetch) ? Tb >> 5 : 0;
  int ti = 0;
  if (4 < tile_full) {
    float fold[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) fold[r] = 0.0f;
    fold_exchange(fold_request(0), fold);
    // three tiles per trip, the register sets taking turns: (tile, its emissions, the set that
    // receives those of the tile two ahead); all of tiles ti .. ti + 4 must be full
    for (; ti + 4 < tile_full; ti += 3) {
      fast_tile(ti, evA, evC, fold);
      fast_tile(ti + 1, evB, evA, fold);
      fast_tile(ti + 2, evC, evB, fold);
    }
  }
  // what is left: at most five tiles of such a wavefront (the last full ones and the one the
  // utterance ends in), all tiles of the others
  for (; ti < tile_valid; ti += 2) {
    tile(ti, evA, evB);  // (requests the next tile's emissions itself, one tile ahead)
    if (ti + 1 < tile_valid) tile(ti + 1, evB, evA);
  }

  // frames past the utterance: egrads is exactly zero there
  for (int ti = tile_valid; ti < ntiles; ++ti) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int t = ti * 32 + mfma_row(r, h);
      if (t < d.T && vok) stf(eout + (size_t)t * d.V + vcol, 0.0f);
    }
  }

  // pgrads write-out (as pgrads_tile's): delta * (Y * sum), then the row's blank / label totals
#pragma unroll
  for (int mb = 0; mb < NMB; ++mb) mfma_settle(pacc[mb]);
  float praw[NMB][16], mraw[NMB][16];
#pragma unroll
  for (int mb = 0; mb < NMB; ++mb)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int uc = min(32 * mb + mfma_row(r, h), d.U - 1);
      praw[mb][r] = ldf(Pb + (size_t)uc * d.V + vc);
      mraw[mb][r] = mPb[uc];
    }
  __builtin_amdgcn_sched_barrier(0);
  TIO* pout = pgrads + (size_t)b * d.U * d.V;
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int u = 32 * mb + mfma_row(r, h);
      float g = 0.0f;
      if (mb < NMB) {
        const float y = __expf(praw[mb < NMB ? mb : 0][r] - mraw[mb < NMB ? mb : 0][r]);
        g = u < Ub ? y * pacc[mb < NMB ? mb : 0][r] : 0.0f;
      }
      if (u < d.U && vok) {
        float res = delta * g;
        if (vcol == d.blank) res += delta * L.Rt.gB[u];
        else if (vcol == L.Rt.label[u]) res += delta * L.Rt.gL[u];
        stf(pout + (size_t)u * d.V + vcol, res);
      }
    }
}

// grid (column tiles of 128, 1, B); dynamic LDS: sizeof(FusedLds).  Needs U <= 112 (one slice of
// the label axis for egrads, one tile of 128 rows for pgrads) and the blank / label terms
// folded into both write-outs.
template <typename TIO>
__global__ __launch_bounds__(256) void grads_fused_kernel(
    const TIO* __restrict__ E, const TIO* __restrict__ P, const float* __restrict__ mE,
    const float* __restrict__ mP, WImages img, const float* __restrict__ deltas,
    TIO* __restrict__ egrads, TIO* __restrict__ pgrads, const int* __restrict__ inLen,
    const int* __restrict__ labLen, Dims d, int Tw, SparseTerms sp, SparsePTerms spp) {
  extern __shared__ __attribute__((aligned(16))) unsigned char fused_lds_raw[];
  FusedLds& L = *reinterpret_cast<FusedLds*>(fused_lds_raw);
  const int b = blockIdx.z;
  int Tb, Ub;
  utt_extent(inLen, labLen, b, d.T, d.U, Tb, Ub);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col0 = blockIdx.x * 128 + wave * 32;
  if (Tb == 0 || Ub == 0) {  // nothing to contract: both gradients are exactly zero
    for (int t = 0; t < d.T; ++t)
      if (lane < 32 && col0 + lane < d.V) stf(egrads + ((size_t)b * d.T + t) * d.V + col0 + lane, 0.0f);
    for (int u = 0; u < d.U; ++u)
      if (lane < 32 && col0 + lane < d.V) stf(pgrads + ((size_t)b * d.U + u) * d.V + col0 + lane, 0.0f);
    return;
  }
  int nmatch = 0;
  for (int u0 = 0; u0 < Ub - 1; u0 += 64) {
    const int u = u0 + lane;
    const int l = (u < Ub - 1) ? label_at(sp.labels, d, b, u) : -1;
    const bool hit = l >= col0 && l < col0 + 32 && l != d.blank;
    const unsigned long long m = __ballot(hit);
    if (hit) L.Match[wave][nmatch + __popcll(m & ((1ull << lane) - 1))] = (unsigned short)u;
    nmatch += __popcll(m);
  }
  if (threadIdx.x < 128) {
    const int u = threadIdx.x;
    const bool valid = u < Ub, has_label = valid && u + 1 < Ub;
    const int l = has_label ? label_at(spp.labels, d, b, u) : d.blank;
    L.Rt.gB[u] = valid ? spp.gB[(size_t)b * d.Ua + u] : 0.0f;
    L.Rt.gL[u] = has_label ? spp.gL[(size_t)b * d.Ua + u] : 0.0f;
    L.Rt.label[u] = (has_label && l != d.blank) ? l : -1;
  }
  __syncthreads();
#define RNNT_FUSED_WALK(NS, NMB) \
  fused_walk<NS, NMB>(E, P, mE, mP, img, deltas, egrads, pgrads, L, d, Tw, b, Tb, Ub, sp, nmatch)
  if (Ub <= 32) RNNT_FUSED_WALK(2, 1);
  else if (Ub <= 64) RNNT_FUSED_WALK(4, 2);
  else if (Ub <= 80) RNNT_FUSED_WALK(5, 3);
  else if (Ub <= 96) RNNT_FUSED_WALK(6, 3);
  else RNNT_FUSED_WALK(7, 4);
#undef RNNT_FUSED_WALK
}

}  // namespace

// Whether the fused walk can take this shape -- one slice of the label axis, labels to fold the
// blank / label terms for -- and whether it is expected to pay: enough column tiles to fill the
// device with one workgroup per CU (a small grid is better served by the two kernels, whose
// pgrads tiles can share their frames between workgroups), and a vocabulary large enough for
// the folded terms.
bool grads_fused_possible(const Dims& d) {
  return d.U >= 2 && wplane_up(d.U) <= WImages::kCols && d.B > 0 && d.T > 0 && d.V > 0;
}
bool grads_fused_pays(const Dims& d) {
  return d.V >= 512 && (long)((d.V + 127) / 128) * d.B >= 192;
}

template <typename TIO>
static int grads_fused_any(const TIO* E, const TIO* P, const float* mE, const float* mP,
                           const WImages& img, const float* deltas, TIO* egrads, TIO* pgrads,
                           const int* inLen, const int* labLen, const Dims& d,
                           const SparseTerms& sp, const SparsePTerms& spp, hipStream_t s) {
  if (!grads_fused_possible(d)) return fail(kInvalid, "fused gradients: shape not supported");
  if (!sp.labels || !spp.gB || !spp.labels || !img.e || !img.p)
    return fail(kInvalid, "fused gradients: need the W images and the folded blank / label terms");
  static_assert(WImages::kCols == 16 * kEsMaxS, "one slice of the label axis");
  const int Tw = wplane_tw(d.T);
  auto kernel = grads_fused_kernel<TIO>;
  RNNT_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)sizeof(FusedLds)));
  hipLaunchKernelGGL(kernel, dim3((d.V + 127) / 128, 1, d.B), dim3(256), sizeof(FusedLds), s, E, P,
                     mE, mP, img, deltas, egrads, pgrads, inLen, labLen, d, Tw, sp, spp);
  RNNT_LAUNCH_CHECK("grads_fused_kernel");
  return kOk;
}
int launch_grads_fused(const float* E, const float* P, const float* mE, const float* mP,
                       const WImages& img, const float* deltas, float* egrads, float* pgrads,
                       const int* inLen, const int* labLen, const Dims& d, const SparseTerms& sp,
                       const SparsePTerms& spp, hipStream_t s) {
  return grads_fused_any(E, P, mE, mP, img, deltas, egrads, pgrads, inLen, labLen, d, sp, spp, s);
}

}  // namespace rnnt
