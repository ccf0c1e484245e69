// Streaming forms of the two dense-gradient contractions (transducer/torch_binding.py:85-89)
// for gfx950.  Products are formed on the bf16 matrix cores from exact three-way splits of the
// fp32 operands (rnnt_split.h).  Both kernels keep the vocabulary-side operand in REGISTERS,
// read straight from global memory in the instruction's own lane order (32 consecutive v per
// half-wave = one 128-byte line), and pass only the small W operand through LDS:
//
//   egrads[t,v] = delta * exp(E[t,v]-mE[t]) * sum_u Wn[t,u] * Y[u,v]      Y = exp(P-mP)
//       a wavefront owns 32 columns v and holds Y[:, its columns] (all label positions) in
//       registers for its whole life; it walks the frames 32 at a time, reads the 32 x U slab
//       of W from LDS, and multiplies the finished 32x32 block with exp(E-mE) on its way out.
//       E is read once and egrads written once, each as whole cache lines.
//
//   pgrads[u,v] = delta * exp(P[u,v]-mP[u]) * sum_t Wt[u,t] * X[t,v]      X = exp(E-mE)
//       a wavefront owns 32 columns v and all (up to 128) label positions; it walks the frames
//       32 at a time, turning the 32 x 32 slab of E it just loaded into X in registers.
//
// v_mfma_f32_32x32x16_bf16 takes, per lane, eight consecutive k of its row (A) or column (B):
// k = 8*(lane/32) + i.  A lane reads them with one 16-byte LDS load per piece.
#include <algorithm>
#include <type_traits>

#include "rnnt_internal.h"
#include "rnnt_io.h"
#include "rnnt_split.h"
#include "rnnt_grads.h"

// This file is compiled in six parts side by side (-DRNNT_GRADS_PART=0..5: egrads then pgrads,
// each for fp32, bf16 and fp16 scores; a part instantiates only its own kernels), or whole when
// the macro is not given.
#ifndef RNNT_GRADS_PART
#define RNNT_GRADS_PART -1
#endif
#define RNNT_IN_PART(n) (RNNT_GRADS_PART < 0 || RNNT_GRADS_PART == (n))

namespace rnnt {

namespace {


// ------------------------------------------------------------------ egrads

// Which of two register sets a tile of the egrads walk works on (chosen at compile time).
__device__ __forceinline__ float (&pick_set(std::true_type, float (&a)[16], float (&)[16]))[16] {
  return a;
}
__device__ __forceinline__ float (&pick_set(std::false_type, float (&)[16], float (&b)[16]))[16] {
  return b;
}

struct SlabRegs {
  float4 v0, v1, v2, v3;
  float m;
};

// The frames one egrads launch covers and where they go: tiles [tile_begin, tile_end) of 32
// frames; frame t of utterance b lands in row b * out_T + (t - t_base) of the output array.  The
// whole frame axis into the caller's array: {0, tiles of T, T, 0}.
struct EgradsWindow {
  int tile_begin, tile_end, out_T, t_base;
};

// The walk of one workgroup over its frame tiles with NS steps of sixteen label positions
// (a template parameter, so the matrix instructions of a tile form one straight-line block).
// Label positions past the utterance contribute exact zeros: their Y rows are masked and the
// W slab is zero there.
// kMode: what a launch does with the sums of its slice of the label axis.
//   kEgWhole    out = delta (X sums + sparse terms)         the only slice
//   kEgAdd      out = delta (out + X sums)                  onto what the caller's array holds
//   kEgPartial  out = sums (first slice) or out + sums      a slice but the last of several:
//                                                           no emissions read, no exponentials
//   kEgFinal    out = delta (X (out + sums) + sparse terms) the last of several slices
constexpr int kEgWhole = 0, kEgAdd = 1, kEgPartial = 2, kEgFinal = 3;
// kManyLabels: compiled for transcripts that put more than two labels into most blocks of 32
// columns (the launcher decides by U * 32 > 2 V); see where the terms are fetched.
template <int NS, int kMode, bool kManyLabels, typename TIO, typename TOUT>
__device__ __forceinline__ void egrads_walk(
    const TIO* __restrict__ E, const TIO* __restrict__ P, const float* __restrict__ mE,
    const float* __restrict__ mP, const float* __restrict__ Wn, const float* __restrict__ deltas,
    TOUT* __restrict__ egrads, unsigned short (*As)[3][kEsPlane], float (*Ms)[32], const Dims& d,
    int Up, int Tw, int tiles_per_chunk, int u_lo, int b, int Tb, int Ub, const SparseTerms& sp,
    const unsigned short* match, int nmatch, float (*Sp)[32], const EgradsWindow& win) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, h = lane >> 5;
  const int wave_col0 = blockIdx.x * 128 + wave * 32;  // this wavefront's 32 columns
  const int vcol = wave_col0 + l32;
  const bool vok = vcol < d.V;
  const int vc = vok ? vcol : d.V - 1;  // always readable
  const bool cols_full = wave_col0 + 32 <= d.V;
  // lane that owns the blank column, if it is one of this wavefront's and terms are folded in
  constexpr bool kSparse = kMode == kEgWhole || kMode == kEgFinal;  // may fold sparse terms in
  constexpr bool kScores = kMode != kEgPartial;                     // reads the emissions
  // reads what the output holds (a first partial slice starts from nothing)
  const bool reads_out = kMode == kEgAdd || kMode == kEgFinal || (kMode == kEgPartial && u_lo > 0);
  const int blank_lane = (sp.labels && d.blank >= wave_col0 && d.blank < wave_col0 + 32)
                             ? d.blank - wave_col0 : -1;
  const int tile_lo = win.tile_begin + blockIdx.y * tiles_per_chunk;
  const int tile_hi = min(tile_lo + tiles_per_chunk, win.tile_end);
  const int tile_valid = min(tile_hi, (Tb + 31) >> 5);  // tiles that hold frames of the utterance
  const float delta = deltas ? deltas[b] : 1.0f;
  const TIO* Eb = E + (size_t)b * d.T * d.V;
  // frame t of the utterance is row t - win.t_base of its block of win.out_T rows in `egrads`
  TOUT* out = egrads + (size_t)b * win.out_T * d.V;
  const float* mEb = mE + (size_t)b * d.T;

  // Y fragments for this wavefront's columns (branch-free: clamped address, masked value):
  // step s holds label positions u_lo + 16 s + 8 h + i, split into their three bf16 pieces
  Frag3 Yf[NS];
  if (tile_lo < tile_valid) {
    const TIO* Pb = P + (size_t)b * d.U * d.V;
    const float* mPb = mP + (size_t)b * d.U;
    // (all scores and row maxima are requested before the first is used: step by step, each
    // step's loads are waited for before the next step's are issued)
    float praw[NS][8], mraw[NS][8];
#pragma unroll
    for (int s = 0; s < NS; ++s)
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int u = u_lo + 16 * s + 8 * h + i;
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
        const int u = u_lo + 16 * s + 8 * h + i;
        const float e = __expf(praw[s][i] - mraw[s][i]);
        y[i] = (u < Ub && vok) ? e : 0.0f;
      }
      Yf[s] = split8(y);
    }
  }

  // W slab staging: columns u_lo .. u_lo + 16 NS of the 32 x Up slab of frame tile ti (all of
  // it when the label axis fits one launch), float4 by float4, each split into its three pieces
  // on the way into LDS
  const int up4 = Up >> 2, lo4 = u_lo >> 2, cw4 = min(Up - u_lo, 16 * kEsMaxS) >> 2;
  const int nvec = 32 * cw4;
  int lds_off[4], src_idx[4];
  bool vec_ok[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int idx = tid + 256 * i;
    vec_ok[i] = idx < nvec;
    const int ic = vec_ok[i] ? idx : nvec - 1;  // loads stay unconditional, stores are masked
    src_idx[i] = (ic / cw4) * up4 + lo4 + ic % cw4;
    lds_off[i] = vec_ok[i] ? (idx / cw4) * kEsPitch + 4 * (idx % cw4) : 0;
  }
  // per-lane part of the element offset inside a tile; the per-register part is r-dependent
  // only through compile-time multiples of V
  const unsigned lane_off = (unsigned)(4 * h) * (unsigned)d.V + (unsigned)vcol;
  auto fetch_slab = [&](int ti) -> SlabRegs {
    const float4* src =
        reinterpret_cast<const float4*>(Wn + ((size_t)b * Tw + (size_t)ti * 32) * Up);
    SlabRegs s;
    s.v0 = src[src_idx[0]];
    s.v1 = src[src_idx[1]];
    s.v2 = src[src_idx[2]];
    s.v3 = src[src_idx[3]];
    s.m = mEb[min(ti * 32 + (tid & 31), Tb - 1)];
    return s;
  };
  auto store_slab = [&](int buf, const SlabRegs& s) {
    const float4 v[4] = {s.v0, s.v1, s.v2, s.v3};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      uint2 ph, pm, pl;
      split_pair(v[i].x, v[i].y, ph.x, pm.x, pl.x);
      split_pair(v[i].z, v[i].w, ph.y, pm.y, pl.y);
      if (vec_ok[i]) {
        *reinterpret_cast<uint2*>(&As[buf][0][lds_off[i]]) = ph;
        *reinterpret_cast<uint2*>(&As[buf][1][lds_off[i]]) = pm;
        *reinterpret_cast<uint2*>(&As[buf][2][lds_off[i]]) = pl;
      }
    }
    if (tid < 32) Ms[buf][tid] = s.m * kLog2e;
  };

  int cur = 0;
  if (tile_lo < tile_valid) store_slab(0, fetch_slab(tile_lo));
  __syncthreads();

  // the first kEsPrefetch matches, resolved once: label position and target lane
  int mu[kEsPrefetch], mc[kEsPrefetch];
#pragma unroll
  for (int i = 0; i < kEsPrefetch; ++i) {
    mu[i] = (sp.labels && i < nmatch) ? match[i] : 0;
    mc[i] = (sp.labels && i < nmatch) ? label_at(sp.labels, d, b, mu[i]) - wave_col0 : -1;
  }

  // bf16 only: with half the bytes the kernel is held by how long a request takes, not by how
  // many bytes move, so a tile's emissions are requested one whole tile before their use
  // (1.06 -> 0.94 ms).  In fp32 it runs at the speed of a plain copy of the same arrays and more
  // requests in flight only lengthen the queues (1.11 -> 1.14 ms): there a tile's emissions are
  // requested at its own start and arrive under its matrix work.
  constexpr bool kAhead = sizeof(TIO) == 2;
  auto load_e = [&](int ti, float (&e)[16]) __attribute__((always_inline)) {
    const int t0 = ti * 32;
    if (cols_full && (t0 + 32 <= Tb)) {
      const TIO* Etile = Eb + (size_t)t0 * d.V;
#pragma unroll
      for (int r = 0; r < 16; ++r)
        e[r] = ldf(Etile + (lane_off + (unsigned)(8 * (r >> 2) + (r & 3)) * (unsigned)d.V));
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r)
        e[r] = ldf(Eb + (size_t)min(t0 + mfma_row(r, h), Tb - 1) * d.V + vc);
    }
  };
  // One tile.  ahead: `evc` holds its emissions and `evn` receives the next tile's.
  auto tile = [&](int ti, float (&evc)[16], float (&evn)[16], auto ahead)
                  __attribute__((always_inline)) {
    const int t0 = ti * 32;
    // the next slab, requested now (the last tile re-reads its own: no branch around the loads)
    const SlabRegs nxt = fetch_slab(min(ti + 1, tile_valid - 1));
    const bool interior = cols_full && (t0 + 32 <= Tb);  // no row or column needs a guard
    const TIO* Etile = Eb + (size_t)t0 * d.V;
    TOUT* Otile = out + (size_t)(t0 - win.t_base) * d.V;
    float evl[16];
    float (&ev)[16] = pick_set(ahead, evc, evl);
    if constexpr (!kScores) {
    } else if constexpr (decltype(ahead)::value) {
      load_e(min(ti + 1, tile_valid - 1), evn);
    } else if (interior) {
      // the emissions of this tile, requested before the matrix work so they arrive under it
#pragma unroll
      for (int r = 0; r < 16; ++r)
        ev[r] = ldf(Etile + (lane_off + (unsigned)(8 * (r >> 2) + (r & 3)) * (unsigned)d.V));
    } else {
      // rows past the utterance are read from its last frame and masked on the way out
#pragma unroll
      for (int r = 0; r < 16; ++r)
        ev[r] = ldf(Eb + (size_t)min(t0 + mfma_row(r, h), Tb - 1) * d.V + vc);
    }
    // a later slice of a long label axis adds to what the earlier ones left: requested here
    // too (asked for at the store, every tile waited a memory round trip for them: 0.44 ms a
    // slice of 112 label positions at B=8 T=10000 V=1000, where the first slice takes 0.30)
    float ov[16];
    if constexpr (kMode != kEgWhole) {
      if (!reads_out) {
#pragma unroll
        for (int r = 0; r < 16; ++r) ov[r] = 0.0f;
      } else if (interior) {
#pragma unroll
        for (int r = 0; r < 16; ++r)
          ov[r] = ldf(Otile + (lane_off + (unsigned)(8 * (r >> 2) + (r & 3)) * (unsigned)d.V));
      } else {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int t = t0 + mfma_row(r, h);
          ov[r] = (t < d.T && vok) ? ldf(out + (size_t)(t - win.t_base) * d.V + vcol) : 0.0f;
        }
      }
    }
    // sparse terms of this tile for up to kEsPrefetch labels that fall into this wavefront's
    // columns: one coalesced load per plane, requested here so it arrives under the matrix work
    float sd[kEsPrefetch], sbl = 0.0f;
    if (kSparse && (nmatch > 0 || blank_lane >= 0)) {
      const int tr = min(t0 + l32, Tb - 1);
#pragma unroll
      for (int i = 0; i < kEsPrefetch; ++i) {
        sd[i] = sp.emT[((size_t)b * d.U + mu[i]) * d.T + tr];
      }
      if (blank_lane >= 0) sbl = sp.bsum[(size_t)b * d.T + tr];
    }
    // two accumulators, so that consecutive matrix instructions never wait on each other
    floatx16 acc, acc2;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = acc2[r] = 0.0f;
    __builtin_amdgcn_sched_barrier(0);
    {
      const unsigned short* arow = &As[cur][0][l32 * kEsPitch + 8 * h];
      uint4 ah[NS], am[NS], al[NS];
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        ah[s] = *reinterpret_cast<const uint4*>(arow + 16 * s);
        am[s] = *reinterpret_cast<const uint4*>(arow + kEsPlane + 16 * s);
        al[s] = *reinterpret_cast<const uint4*>(arow + 2 * kEsPlane + 16 * s);
      }
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        acc = mfma_bf16(al[s], Yf[s].h, acc);
        acc2 = mfma_bf16(ah[s], Yf[s].l, acc2);
        acc = mfma_bf16(am[s], Yf[s].m, acc);
        acc2 = mfma_bf16(am[s], Yf[s].h, acc2);
        acc = mfma_bf16(ah[s], Yf[s].m, acc);
        acc2 = mfma_bf16(ah[s], Yf[s].h, acc2);
      }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] += acc2[r];
    float v[16];
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const float4 m4 = *reinterpret_cast<const float4*>(&Ms[cur][8 * g + 4 * h]);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const int r = 4 * g + k;
        float x;
        if constexpr (kMode == kEgPartial) x = ov[r] + acc[r];
        else if constexpr (kMode == kEgFinal) x = exp_minus_scaled(ev[r], f4at(m4, k)) * (ov[r] + acc[r]);
        else x = exp_minus_scaled(ev[r], f4at(m4, k)) * acc[r];
        v[r] = (interior || t0 + mfma_row(r, h) < Tb) ? x : 0.0f;
      }
    }
    if (kSparse && (nmatch > 0 || blank_lane >= 0)) {  // uniform per wavefront, and rare
      // Lane l32 holds the term of frame t0+l32 (fetched before the matrix block).  The terms go
      // through a per-wavefront LDS strip; the two lanes that own the target column read their
      // 16 frames back as four 16-byte loads.
      const bool row_ok = t0 + l32 < Tb;
      float* strip = &Sp[0][0];
      auto apply = [&](float term, int col, float sign) {
        if (h == 0) strip[l32] = term;
        if (l32 == col) {
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const float4 x = *reinterpret_cast<const float4*>(&strip[8 * g + 4 * h]);
            v[4 * g + 0] += sign * x.x;
            v[4 * g + 1] += sign * x.y;
            v[4 * g + 2] += sign * x.z;
            v[4 * g + 3] += sign * x.w;
          }
        }
      };
#pragma unroll
      for (int i = 0; i < kEsPrefetch; ++i)
        if (i < nmatch) apply(row_ok ? sd[i] : 0.0f, mc[i], -1.0f);
      // more labels in one 32-column block
      if constexpr (kManyLabels) {
        // long transcripts over a small vocabulary (400 labels and 1000 columns put a dozen into
        // every block): their terms are asked for four at a time, so that a tile waits one
        // memory round trip per four, not one per label (B=8 T=10000 U=400 V=1000: 1.21 ->
        // 1.02 ms).  A kernel of its own: compiled into the kernel of the large vocabularies,
        // where it hardly ever runs, it cost that one 1 % (B=32 T=2000 U=100 V=10000).
        constexpr int kBatch = 4;
        for (int i0 = kEsPrefetch; i0 < nmatch; i0 += kBatch) {
          float term[kBatch];
          int col[kBatch];
#pragma unroll
          for (int k = 0; k < kBatch; ++k) {
            const int u = match[min(i0 + k, nmatch - 1)];
            term[k] = sp.emT[((size_t)b * d.U + u) * d.T + min(t0 + l32, Tb - 1)];
            col[k] = label_at(sp.labels, d, b, u) - wave_col0;
          }
#pragma unroll
          for (int k = 0; k < kBatch; ++k)
            if (i0 + k < nmatch) apply(row_ok ? term[k] : 0.0f, col[k], -1.0f);
        }
      } else {
        for (int i = kEsPrefetch; i < nmatch; ++i) {
          const int u = match[i];
          apply(row_ok ? sp.emT[((size_t)b * d.U + u) * d.T + min(t0 + l32, Tb - 1)] : 0.0f,
                label_at(sp.labels, d, b, u) - wave_col0, -1.0f);
        }
      }
      if (blank_lane >= 0) apply(row_ok ? sbl : 0.0f, blank_lane, 1.0f);
    }
    if (interior) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        TOUT* o = Otile + (lane_off + (unsigned)(8 * (r >> 2) + (r & 3)) * (unsigned)d.V);
        if constexpr (kMode == kEgAdd) stf(o, delta * (ov[r] + v[r]));
        else if constexpr (kMode == kEgPartial) stf(o, v[r]);
        else stf(o, delta * v[r]);
      }
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int t = t0 + mfma_row(r, h);
        if (t < d.T && vok) {
          TOUT* o = out + (size_t)(t - win.t_base) * d.V + vcol;
          if constexpr (kMode == kEgAdd) stf(o, delta * (ov[r] + v[r]));
          else if constexpr (kMode == kEgPartial) stf(o, v[r]);
          else stf(o, delta * v[r]);
        }
      }
    }
    store_slab(cur ^ 1, nxt);
    __syncthreads();
    cur ^= 1;
  };
  float evA[16], evB[16];
  if constexpr (kAhead && kScores) {
    // two tiles per trip, the two register sets swapping roles (a copy from one set to the other
    // would wait for the requests a tile too early)
    if (tile_lo < tile_valid) load_e(tile_lo, evA);
    for (int ti = tile_lo; ti < tile_valid; ti += 2) {
      tile(ti, evA, evB, std::true_type());
      if (ti + 1 < tile_valid) tile(ti + 1, evB, evA, std::true_type());
    }
  } else {
    for (int ti = tile_lo; ti < tile_valid; ++ti) tile(ti, evA, evB, std::false_type());
  }

  // frames past the utterance: the dense part is exactly zero (of several slices the first
  // writes the zeros and the later ones leave them)
  if (kMode == kEgWhole || kMode == kEgAdd || (kMode == kEgPartial && u_lo == 0)) {
    for (int ti = max(tile_lo, tile_valid); ti < tile_hi; ++ti) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int t = ti * 32 + mfma_row(r, h);
        if (t < d.T && vok) {
          TOUT* o = out + (size_t)(t - win.t_base) * d.V + vcol;
          stf(o, kMode == kEgAdd ? delta * ldf(o) : 0.0f);
        }
      }
    }
  }
}

template <int kMode, bool kManyLabels, typename TIO, typename TOUT>
__global__ __launch_bounds__(256, 2) void egrads_stream_kernel(
    const TIO* __restrict__ E, const TIO* __restrict__ P, const float* __restrict__ mE,
    const float* __restrict__ mP, const float* __restrict__ Wn, const float* __restrict__ deltas,
    TOUT* __restrict__ egrads, const int* __restrict__ inLen, const int* __restrict__ labLen,
    Dims d, int Up, int Tw, int tiles_per_chunk, int u_lo, SparseTerms sp, EgradsWindow win) {
  __shared__ __attribute__((aligned(16))) unsigned short As[2][3][kEsPlane];
  __shared__ __attribute__((aligned(16))) float Ms[2][32];  // mE * log2(e) of the slab's frames
  __shared__ __attribute__((aligned(16))) float Strip[4][32];  // per wavefront: sparse terms
  __shared__ unsigned short Match[4][kMaxLabels];  // per wavefront: label positions whose label
                                                   // is one of its 32 columns
  const int b = blockIdx.z;
  int Tb, Ub;
  utt_extent(inLen, labLen, b, d.T, d.U, Tb, Ub);
  // a later slice of the label axis that lies past this utterance adds nothing; only the last
  // slice (the one that is given the factors) still has to finish what is there
  if (kMode == kEgPartial && u_lo > 0 && u_lo >= Ub) return;
  if (kMode == kEgAdd && u_lo > 0 && u_lo >= Ub && deltas == nullptr) return;
  int nmatch = 0;
  if (sp.labels) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col0 = blockIdx.x * 128 + wave * 32;
    for (int u0 = 0; u0 < Ub - 1; u0 += 64) {
      const int u = u0 + lane;
      const int l = (u < Ub - 1) ? label_at(sp.labels, d, b, u) : -1;
      const bool hit = l >= col0 && l < col0 + 32 && l != d.blank;
      const unsigned long long m = __ballot(hit);
      if (hit) Match[wave][nmatch + __popcll(m & ((1ull << lane) - 1))] = (unsigned short)u;
      nmatch += __popcll(m);
    }
  }
  // columns of the slab past Up are never staged; clear them once so that a walk that rounds
  // its step count up multiplies zeros there, not whatever the LDS held
  for (int e = threadIdx.x; e < 3 * kEsPlane; e += 256)
    reinterpret_cast<unsigned*>(&As[0][0][0])[e] = 0u;
  __syncthreads();
  const int nsteps = (min(max(Ub - u_lo, 0), 16 * kEsMaxS) + 15) >> 4;
#define RNNT_EG_WALK(NS)                                                                      \
  egrads_walk<NS, kMode, kManyLabels>(E, P, mE, mP, Wn, deltas, egrads, As, Ms, d, Up, Tw,   \
                               tiles_per_chunk, u_lo, b, Tb, Ub, sp, Match[threadIdx.x >> 6], \
                               nmatch, &Strip[threadIdx.x >> 6], win)
  if (nsteps <= 2) RNNT_EG_WALK(2);
  else if (nsteps <= 4) RNNT_EG_WALK(4);
  else if (nsteps == 5) RNNT_EG_WALK(5);
  else if (nsteps == 6) RNNT_EG_WALK(6);
  else RNNT_EG_WALK(7);
#undef RNNT_EG_WALK
}

// ------------------------------------------------------------------ pgrads

// Splitting a tile's frames over several workgroups (small grids: one utterance with a small
// vocabulary is a single tile, whose workgroup would walk all frames alone).  Workgroup c of
// `chunks` sums slabs [c*per, (c+1)*per) and leaves its sums in `partial`; the one that arrives
// last at the tile's counter adds all of them up in chunk order (so the result does not depend
// on who was last) and writes the tile.  Nobody waits for anybody.  per == kPsFlush, always:
// see pgrads_split_plan.
struct PSplit {
  int chunks = 1, per = 0;
  float* partial = nullptr;  // [tile][chunk][4 blocks][16 registers][256 threads]
  int* counter = nullptr;    // [tile], zero before the launch
};
constexpr int kPsPartialFloats = 4 * 16 * 256;

// One workgroup's 128 x 128 tile with NMB 32-row blocks of label positions in use (a template
// parameter, so the matrix instructions of a slice form one straight-line block).  Products are
// formed on the bf16 matrix cores from exact three-way splits of both operands (rnnt_split.h).
template <int NMB, bool kAccumulate, bool kSplit, typename TIO>
__device__ __forceinline__ void pgrads_tile(
    const TIO* __restrict__ E, const TIO* __restrict__ P, const float* __restrict__ mE,
    const float* __restrict__ mP, const float* __restrict__ Wt, const float* __restrict__ deltas,
    TIO* __restrict__ pgrads, unsigned short (*As)[3][kPsPlane], float (*Ms)[32], const Dims& d,
    int Up, int Tw, int b, int u0, int Tb, int Ub, const PRowTerms* rt, const PSplit& split,
    int chunk, int tile, int* last_flag) {
  if (kSplit && NMB == 0 && chunk > 0) return;  // nothing to sum: chunk 0 alone writes the zeros
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, h = lane >> 5;
  const int vcol = blockIdx.x * 128 + wave * 32 + l32;
  const bool vok = vcol < d.V;
  const int vc = vok ? vcol : d.V - 1;
  const float delta = deltas ? deltas[b] : 1.0f;
  TIO* out = pgrads + (size_t)b * d.U * d.V;

  // The matrix instruction truncates what falls below its accumulator's last bit, so a long
  // running sum drifts low; every kPsFlush slabs it is added (vector ALU, round to nearest)
  // into a second accumulator and restarted.
  floatx16 acc[NMB > 0 ? NMB : 1], tot[NMB > 0 ? NMB : 1];
#pragma unroll
  for (int mb = 0; mb < NMB; ++mb)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[mb][r] = tot[mb][r] = 0.0f;

  if (NMB > 0) {
    const TIO* Eb = E + (size_t)b * d.T * d.V;
    const float* mEb = mE + (size_t)b * d.T;
    // W^T slab staging: 128 rows (u) x 32 frames = 1024 float4, four per thread; rows past the
    // padded label axis re-read its last row (their blocks are never multiplied)
    const int arow = tid >> 3, ac4 = tid & 7;  // rows arow + 32*i, frames 4*ac4 .. +3
    const float* asrc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
      asrc[i] = Wt + ((size_t)b * Up + min(u0 + arow + 32 * i, Up - 1)) * Tw + 4 * ac4;
    struct XRegs { float v[2][8]; };
    auto fetch_slab = [&](int k0) -> SlabRegs {
      SlabRegs s;
      s.v0 = *reinterpret_cast<const float4*>(asrc[0] + k0);
      s.v1 = *reinterpret_cast<const float4*>(asrc[1] + k0);
      s.v2 = *reinterpret_cast<const float4*>(asrc[2] + k0);
      s.v3 = *reinterpret_cast<const float4*>(asrc[3] + k0);
      s.m = mEb[min(k0 + (tid & 31), Tb - 1)];
      return s;
    };
    // frames this lane feeds to the matrix instruction of k-step s: k0 + 16 s + 8 h + i
    auto fetch_x = [&](int k0) -> XRegs {
      XRegs x;
#pragma unroll
      for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int t = min(k0 + 16 * s + 8 * h + i, Tb - 1);
          x.v[s][i] = ldf(Eb + (size_t)t * d.V + vc);
        }
      return x;
    };
    auto store_slab = [&](int buf, const SlabRegs& s) {
      const float4 v[4] = {s.v0, s.v1, s.v2, s.v3};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        uint2 ph, pm, pl;
        split_pair(v[i].x, v[i].y, ph.x, pm.x, pl.x);
        split_pair(v[i].z, v[i].w, ph.y, pm.y, pl.y);
        const int o = (arow + 32 * i) * kPsPitch + 4 * ac4;
        *reinterpret_cast<uint2*>(&As[buf][0][o]) = ph;
        *reinterpret_cast<uint2*>(&As[buf][1][o]) = pm;
        *reinterpret_cast<uint2*>(&As[buf][2][o]) = pl;
      }
      if (tid < 32) Ms[buf][tid] = s.m * kLog2e;
    };

    const int nk_all = (Tb + 31) >> 5;
    const int k_lo = kSplit ? min(chunk * split.per, nk_all) : 0;
    const int nk = kSplit ? min(k_lo + split.per, nk_all) : nk_all;  // one past the last slab
    const int k_first = min(k_lo, nk_all - 1);  // (a chunk past the utterance loads, sums nothing)
    store_slab(0, fetch_slab(k_first * 32));
    XRegs xr = fetch_x(k_first * 32);
    __syncthreads();
    int cur = 0;
    for (int kt = k_lo; kt < nk; ++kt) {
      // X = exp(E - mE) for this slab (finite everywhere; W^T is zero past the utterance and
      // columns past V are dropped on the way out), split into its three pieces in the
      // instruction's operand layout
      Frag3 xb[2];
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const float4 ma = *reinterpret_cast<const float4*>(&Ms[cur][16 * s + 8 * h]);
        const float4 mb4 = *reinterpret_cast<const float4*>(&Ms[cur][16 * s + 8 * h + 4]);
        float x[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float m = i < 4 ? f4at(ma, i) : f4at(mb4, i - 4);
          x[i] = exp_minus_scaled(xr.v[s][i], m);  // frames past the utterance repeat its last one
        }
        xb[s] = split8(x);
      }
      // the next slab, requested now (the last step re-reads its own: no branch around the loads)
      const int knext = min(kt + 1, nk - 1) * 32;
      const SlabRegs nxt = fetch_slab(knext);
      xr = fetch_x(knext);
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        uint4 ah[NMB > 0 ? NMB : 1], am[NMB > 0 ? NMB : 1], al[NMB > 0 ? NMB : 1];
#pragma unroll
        for (int mb = 0; mb < NMB; ++mb) {
          const int o = (32 * mb + l32) * kPsPitch + 16 * s + 8 * h;
          ah[mb] = *reinterpret_cast<const uint4*>(&As[cur][0][o]);
          am[mb] = *reinterpret_cast<const uint4*>(&As[cur][1][o]);
          al[mb] = *reinterpret_cast<const uint4*>(&As[cur][2][o]);
        }
        // six piece products per block, smallest first; blocks interleaved so that consecutive
        // instructions never wait on each other's accumulator
#pragma unroll
        for (int mb = 0; mb < NMB; ++mb) acc[mb] = mfma_bf16(al[mb], xb[s].h, acc[mb]);
#pragma unroll
        for (int mb = 0; mb < NMB; ++mb) acc[mb] = mfma_bf16(ah[mb], xb[s].l, acc[mb]);
#pragma unroll
        for (int mb = 0; mb < NMB; ++mb) acc[mb] = mfma_bf16(am[mb], xb[s].m, acc[mb]);
#pragma unroll
        for (int mb = 0; mb < NMB; ++mb) acc[mb] = mfma_bf16(am[mb], xb[s].h, acc[mb]);
#pragma unroll
        for (int mb = 0; mb < NMB; ++mb) acc[mb] = mfma_bf16(ah[mb], xb[s].m, acc[mb]);
#pragma unroll
        for (int mb = 0; mb < NMB; ++mb) acc[mb] = mfma_bf16(ah[mb], xb[s].h, acc[mb]);
      }
      if ((kt - k_lo + 1) % kPsFlush == 0) {
#pragma unroll
        for (int mb = 0; mb < NMB; ++mb)
#pragma unroll
          for (int r = 0; r < 16; ++r) { tot[mb][r] += acc[mb][r]; acc[mb][r] = 0.0f; }
      }
      store_slab(cur ^ 1, nxt);
      __syncthreads();
      cur ^= 1;
    }
  }
#pragma unroll
  for (int mb = 0; mb < NMB; ++mb)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[mb][r] += tot[mb][r];

  if (kSplit && NMB > 0) {
    float* mine = split.partial + ((size_t)tile * split.chunks + chunk) * kPsPartialFloats;
#pragma unroll
    for (int mb = 0; mb < NMB; ++mb)
#pragma unroll
      for (int r = 0; r < 16; ++r) mine[(mb * 16 + r) * 256 + tid] = acc[mb][r];
    __threadfence();  // the sums are out before the arrival is counted
    __syncthreads();
    if (tid == 0) {
      const int before = __hip_atomic_fetch_add(&split.counter[tile], 1, __ATOMIC_ACQ_REL,
                                                __HIP_MEMORY_SCOPE_AGENT);
      *last_flag = before == split.chunks - 1;
    }
    __syncthreads();
    if (!*last_flag) return;
    __threadfence();  // the others' sums are visible after their arrivals were seen
    const float* all = split.partial + (size_t)tile * split.chunks * kPsPartialFloats;
#pragma unroll
    for (int mb = 0; mb < NMB; ++mb)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[mb][r] = 0.0f;
    for (int c = 0; c < split.chunks; ++c) {
      const float* src = all + (size_t)c * kPsPartialFloats;
#pragma unroll
      for (int mb = 0; mb < NMB; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          acc[mb][r] += __builtin_nontemporal_load(&src[(mb * 16 + r) * 256 + tid]);
    }
  }

  const TIO* Pb = P + (size_t)b * d.U * d.V;
  const float* mPb = mP + (size_t)b * d.U;
  // The tile's own scores and row maxima, ALL requested before the first is used: written as
  // one loop the compiler waits for every load right where it is issued (the store before it
  // included), and the write-out of a tile is 64 memory round trips in a row, a fifth of the
  // kernel's time at 2000 frames.
  float praw[NMB > 0 ? NMB : 1][16], mraw[NMB > 0 ? NMB : 1][16];
#pragma unroll
  for (int mb = 0; mb < NMB; ++mb)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int uc = min(u0 + 32 * mb + mfma_row(r, h), d.U - 1);
      praw[mb][r] = ldf(Pb + (size_t)uc * d.V + vc);
      mraw[mb][r] = mPb[uc];
    }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int u = u0 + 32 * mb + mfma_row(r, h);
      float g = 0.0f;
      if (mb < NMB) {
        const float y = __expf(praw[mb < NMB ? mb : 0][r] - mraw[mb < NMB ? mb : 0][r]);
        g = u < Ub ? y * acc[mb < NMB ? mb : 0][r] : 0.0f;
      }
      if (u < d.U && vok) {
        TIO* o = out + (size_t)u * d.V + vcol;
        float res = delta * (kAccumulate ? ldf(o) + g : g);
        if (!kAccumulate && rt != nullptr) {
          // the blank / label terms of this row (what sparse_p_kernel adds), same arithmetic:
          // delta * dense, then + delta * term.  Read from LDS with one address per half-wave.
          const int k = 32 * mb + mfma_row(r, h);
          if (vcol == d.blank) res += delta * rt->gB[k];
          else if (vcol == rt->label[k]) res += delta * rt->gL[k];
        }
        stf(o, res);
      }
    }
}

template <bool kAccumulate, bool kSplit, typename TIO>
__global__ __launch_bounds__(256, 2) void pgrads_stream_kernel(
    const TIO* __restrict__ E, const TIO* __restrict__ P, const float* __restrict__ mE,
    const float* __restrict__ mP, const float* __restrict__ Wt, const float* __restrict__ deltas,
    TIO* __restrict__ pgrads, const int* __restrict__ inLen, const int* __restrict__ labLen,
    Dims d, int Up, int Tw, SparsePTerms sp, PSplit split) {
  __shared__ __attribute__((aligned(16))) unsigned short As[2][3][kPsPlane];
  __shared__ __attribute__((aligned(16))) float Ms[2][32];
  __shared__ PRowTerms Rt;
  __shared__ int last_flag;
  const int b = blockIdx.z;
  const int ut = kSplit ? blockIdx.y / split.chunks : blockIdx.y;
  const int chunk = kSplit ? blockIdx.y - ut * split.chunks : 0;
  const int utiles = kSplit ? gridDim.y / split.chunks : gridDim.y;
  const int tile = (b * utiles + ut) * gridDim.x + blockIdx.x;
  const int u0 = ut * 128;
  int Tb, Ub;
  utt_extent(inLen, labLen, b, d.T, d.U, Tb, Ub);
  const bool folding = !kAccumulate && sp.gB != nullptr;
  if (folding && threadIdx.x < 128) {
    // this tile's rows: blank total, label and label total; rows without one get a label that
    // matches no column.  Visible to all after the barriers of the walk (or the one below).
    const int k = threadIdx.x, u = u0 + k;
    const bool valid = Tb > 0 && u < Ub, has_label = valid && u + 1 < Ub;
    const int l = has_label ? label_at(sp.labels, d, b, u) : d.blank;
    Rt.gB[k] = valid ? sp.gB[(size_t)b * d.Ua + u] : 0.0f;
    Rt.gL[k] = has_label ? sp.gL[(size_t)b * d.Ua + u] : 0.0f;
    Rt.label[k] = (has_label && l != d.blank) ? l : -1;
  }
  if (folding) __syncthreads();
  const PRowTerms* rt = folding ? &Rt : nullptr;
  const int nmb = (u0 < Ub && Tb > 0) ? min(4, (Ub - u0 + 31) >> 5) : 0;  // 32-row blocks in use
#define RNNT_PG_TILE(NMB)                                                                   \
  pgrads_tile<NMB, kAccumulate, kSplit>(E, P, mE, mP, Wt, deltas, pgrads, As, Ms, d, Up, Tw, \
                                        b, u0, Tb, Ub, rt, split, chunk, tile, &last_flag)
  switch (nmb) {
    case 0: RNNT_PG_TILE(0); break;
    case 1: RNNT_PG_TILE(1); break;
    case 2: RNNT_PG_TILE(2); break;
    case 3: RNNT_PG_TILE(3); break;
    default: RNNT_PG_TILE(4); break;
  }
#undef RNNT_PG_TILE
}

}  // namespace

#if RNNT_IN_PART(0)
bool egrads_one_pass(const Dims& d) { return wplane_up(d.U) <= 16 * kEsMaxS; }
#endif

// One pass of the egrads kernels over the frames of `win` (all slices of the label axis), into
// `out` (the caller's array, or a wide copy of a window of it).
template <typename TIO, typename TOUT>
static int egrads_window(const TIO* E, const TIO* P, const float* mE, const float* mP,
                         const float* Wn, const float* deltas, TOUT* out, const int* inLen,
                         const int* labLen, const Dims& d, bool accumulate,
                         const SparseTerms& sparse, const EgradsWindow& win, hipStream_t s) {
  const int Up = wplane_up(d.U), Tw = wplane_tw(d.T);
  const int vtiles = (d.V + 127) / 128, ntiles = win.tile_end - win.tile_begin;
  // enough workgroups to fill 256 CUs two deep several times over, but long enough runs of
  // frames per workgroup to amortise loading the Y fragments
  int chunks = (2048 + vtiles * d.B - 1) / (vtiles * d.B);
  chunks = chunks < 1 ? 1 : chunks;
  const int max_chunks = (ntiles + 7) / 8;
  if (chunks > max_chunks) chunks = max_chunks;
  const int per = (ntiles + chunks - 1) / chunks;
  chunks = (ntiles + per - 1) / per;
  // A launch contracts 16 * kEsMaxS label positions (what a wavefront keeps of Y in registers);
  // a longer label axis goes slice by slice.  Into an array of the caller's that is added to,
  // every slice adds X times its sums and the last one scales the whole.  Otherwise the slices
  // but the last leave their bare sums in the output -- no emissions read, no exponentials --
  // and the last one finishes them: X times the total, the sparse terms, the factor (B=8
  // T=10000 U=400 V=1000, four slices: 1.91 ms with every slice adding X times its sums and
  // asking for the output where it is stored, 1.49 asking for it at the start of a tile).
  const SparseTerms none;
  const int slice = 16 * kEsMaxS;
  const bool many = (long)d.U * 32 > 2 * (long)d.V;  // labels per block of 32 columns
#define RNNT_EG_LAUNCH_(MODE, MANY, DL, SP)                                                   \
  hipLaunchKernelGGL((egrads_stream_kernel<MODE, MANY, TIO, TOUT>), dim3(vtiles, chunks, d.B), \
                     dim3(256), 0, s, E, P, mE, mP, Wn, DL, out, inLen, labLen, d, Up, Tw,    \
                     per, u_lo, SP, win)
  // (only the kernels that fold sparse terms in come in both forms)
#define RNNT_EG_LAUNCH(MODE, DL, SP)                                                          \
  do {                                                                                        \
    if constexpr (sizeof(TOUT) == 2 && MODE != kEgWhole) {                                    \
      /* 16-bit gradients of several slices add up in a wide window: never reached */        \
      return fail(kInvalid, "egrads: slices of 16-bit gradients need a wide window");        \
    } else if constexpr (MODE == kEgWhole || MODE == kEgFinal) {                              \
      if (many) RNNT_EG_LAUNCH_(MODE, true, DL, SP);                                          \
      else RNNT_EG_LAUNCH_(MODE, false, DL, SP);                                              \
    } else {                                                                                  \
      RNNT_EG_LAUNCH_(MODE, false, DL, SP);                                                   \
    }                                                                                         \
  } while (0)
  for (int u_lo = 0; u_lo < Up; u_lo += slice) {
    const bool last = u_lo + slice >= Up;
    if (accumulate) RNNT_EG_LAUNCH(kEgAdd, (last ? deltas : nullptr), none);
    else if (Up <= slice) RNNT_EG_LAUNCH(kEgWhole, deltas, sparse);
    else if (!last) RNNT_EG_LAUNCH(kEgPartial, nullptr, none);
    else RNNT_EG_LAUNCH(kEgFinal, deltas, sparse);
    RNNT_LAUNCH_CHECK("egrads_stream_kernel");
  }
#undef RNNT_EG_LAUNCH
#undef RNNT_EG_LAUNCH_
  return kOk;
}

// rows [t_lo, t_lo + n) of every utterance of dst[B][T][V] = the rows [0, n) of src[B][Tc][V],
// each value rounded once
template <typename TIO>
__global__ void narrow_rows_kernel(const float* __restrict__ src, TIO* __restrict__ dst, int T,
                                   int Tc, int V, int t_lo, int per_row) {
  const int b = blockIdx.y, t = blockIdx.x / per_row;
  const int v = (blockIdx.x - t * per_row) * 256 + threadIdx.x;
  if (v < V) stf(dst + ((size_t)b * T + t_lo + t) * V + v, src[((size_t)b * Tc + t) * V + v]);
}

// `wide`, `wide_bytes`: fp32 scratch for 16-bit gradients whose label axis needs more than one
// slice.  Slices add up in the output array, which for a 16-bit array would round every partial
// sum; so the frames are taken a window at a time, the slices add up in an fp32 copy of the
// window, and the finished window is rounded once on its way into the caller's array.
template <typename TIO>
static int egrads_stream_any(const TIO* E, const TIO* P, const float* mE, const float* mP,
                             const float* Wn, const float* deltas, TIO* egrads, const int* inLen,
                             const int* labLen, const Dims& d, bool accumulate,
                             const SparseTerms& sparse, hipStream_t s, float* wide = nullptr,
                             size_t wide_bytes = 0) {
  if (sparse.labels && accumulate)
    return fail(kInvalid, "sparse-term folding and accumulation are mutually exclusive");
  if (sparse.labels && d.U - 1 > kMaxLabels)  // the per-wavefront match list of the folded terms
    return fail(kInvalid, "egrads: blank/label terms can be folded in for at most %d labels",
                kMaxLabels);
  const int ntiles = (d.T + 31) / 32;
  if (sizeof(TIO) == sizeof(float) || egrads_one_pass(d)) {
    const EgradsWindow all{0, ntiles, d.T, 0};
    return egrads_window(E, P, mE, mP, Wn, deltas, egrads, inLen, labLen, d, accumulate, sparse,
                         all, s);
  }
  if (accumulate) return fail(kInvalid, "egrads: 16-bit gradients cannot be added to");
  const size_t row_bytes = sizeof(float) * (size_t)d.B * d.V;
  const int Tc = (int)std::min<size_t>(wide ? wide_bytes / row_bytes / 32 * 32 : 0, (size_t)ntiles * 32);
  if (Tc < 32)
    return fail(kWorkspace, "egrads: no room for a window of 32 frames of fp32 gradients");
  for (int t_lo = 0; t_lo < d.T; t_lo += Tc) {
    const EgradsWindow win{t_lo / 32, std::min(ntiles, (t_lo + Tc) / 32), Tc, t_lo};
    RNNT_TRY(egrads_window(E, P, mE, mP, Wn, deltas, wide, inLen, labLen, d, false, sparse, win,
                           s));
    const int n = std::min(Tc, d.T - t_lo);
    const unsigned per_row = (unsigned)((d.V + 255) / 256);
    hipLaunchKernelGGL((narrow_rows_kernel<TIO>), dim3(per_row * (unsigned)n, d.B), dim3(256), 0,
                       s, wide, egrads, d.T, Tc, d.V, t_lo, (int)per_row);
    RNNT_LAUNCH_CHECK("narrow_rows_kernel");
  }
  return kOk;
}
#if RNNT_IN_PART(0)
int launch_egrads_stream(const float* E, const float* P, const float* mE, const float* mP,
                         const float* Wn, const float* deltas, float* egrads, const int* inLen,
                         const int* labLen, const Dims& d, bool accumulate,
                         const SparseTerms& sparse, hipStream_t s) {
  return egrads_stream_any(E, P, mE, mP, Wn, deltas, egrads, inLen, labLen, d, accumulate, sparse,
                           s);
}
#endif
#if RNNT_IN_PART(1)
int launch_egrads_stream(const bf16_t* E, const bf16_t* P, const float* mE, const float* mP,
                         const float* Wn, const float* deltas, bf16_t* egrads, const int* inLen,
                         const int* labLen, const Dims& d, bool accumulate,
                         const SparseTerms& sparse, hipStream_t s, float* wide,
                         size_t wide_bytes) {
  return egrads_stream_any(E, P, mE, mP, Wn, deltas, egrads, inLen, labLen, d, accumulate, sparse,
                           s, wide, wide_bytes);
}
#endif
#if RNNT_IN_PART(2)
int launch_egrads_stream(const f16_t* E, const f16_t* P, const float* mE, const float* mP,
                         const float* Wn, const float* deltas, f16_t* egrads, const int* inLen,
                         const int* labLen, const Dims& d, bool accumulate,
                         const SparseTerms& sparse, hipStream_t s, float* wide,
                         size_t wide_bytes) {
  return egrads_stream_any(E, P, mE, mP, Wn, deltas, egrads, inLen, labLen, d, accumulate, sparse,
                           s, wide, wide_bytes);
}
#endif

// Whether the workgroups of a tile share its frames.  A chunk is always kPsFlush slabs, the
// period at which the unsplit walk moves its running sum into the second-level sum: the
// chunks' sums, added in chunk order, then go through exactly the additions the unsplit walk
// performs, so split and unsplit results are the same bits and an utterance's gradient does
// not depend on the batch it is computed in.  Split only when the device would otherwise be
// nearly empty (at most one workgroup per CU after the split): each chunk pays a start-up, a
// device-scope fence and a share of the final addition.
static void pgrads_split_plan(const Dims& d, int& chunks, int& per) {
  const long tiles = (long)((d.V + 127) / 128) * ((d.U + 127) / 128) * d.B;
  const int nk = (d.T + 31) / 32;
  per = kPsFlush;
  chunks = (nk + per - 1) / per;
  if (chunks < 2 || tiles * chunks > 256) chunks = 1;
}

#if RNNT_IN_PART(3)
size_t pgrads_split_bytes(const Dims& d) {
  if (d.B == 0 || d.T == 0 || d.U == 0 || d.V == 0) return 0;
  int chunks, per;
  pgrads_split_plan(d, chunks, per);
  if (chunks <= 1) return 0;
  const size_t tiles = (size_t)((d.V + 127) / 128) * ((d.U + 127) / 128) * d.B;
  return tiles * chunks * kPsPartialFloats * sizeof(float) + ((tiles * sizeof(int) + 255) & ~(size_t)255);
}
#endif

static __global__ void zero_ints_kernel(int* x, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) x[i] = 0;
}

template <typename TIO>
static int pgrads_stream_any(const TIO* E, const TIO* P, const float* mE, const float* mP,
                             const float* Wt, const float* deltas, TIO* pgrads, const int* inLen,
                             const int* labLen, const Dims& d, bool accumulate,
                             const SparsePTerms& sp, void* split_ws, hipStream_t s) {
  if (sp.gB && accumulate)
    return fail(kInvalid, "sparse-term folding and accumulation are mutually exclusive");
  const int Up = wplane_up(d.U), Tw = wplane_tw(d.T);
  const int vtiles = (d.V + 127) / 128, utiles = (d.U + 127) / 128;
  PSplit split;
  if (split_ws != nullptr) pgrads_split_plan(d, split.chunks, split.per);
  if (split.chunks > 1) {
    // counters first (256-byte multiple), partial sums behind them; cleared by a kernel, not a
    // memset node, so that the call can be captured into a graph
    const int tiles = vtiles * utiles * d.B;
    split.counter = static_cast<int*>(split_ws);
    split.partial = reinterpret_cast<float*>(static_cast<char*>(split_ws) +
                                             ((tiles * sizeof(int) + 255) & ~(size_t)255));
    hipLaunchKernelGGL(zero_ints_kernel, dim3((tiles + 255) / 256), dim3(256), 0, s,
                       split.counter, tiles);
    RNNT_LAUNCH_CHECK("zero_ints_kernel");
    const dim3 grid(vtiles, utiles * split.chunks, d.B);
    if (accumulate)
      hipLaunchKernelGGL((pgrads_stream_kernel<true, true, TIO>), grid, dim3(256), 0, s, E, P, mE,
                         mP, Wt, deltas, pgrads, inLen, labLen, d, Up, Tw, sp, split);
    else
      hipLaunchKernelGGL((pgrads_stream_kernel<false, true, TIO>), grid, dim3(256), 0, s, E, P, mE,
                         mP, Wt, deltas, pgrads, inLen, labLen, d, Up, Tw, sp, split);
    RNNT_LAUNCH_CHECK("pgrads_stream_kernel (split)");
    return kOk;
  }
  const dim3 grid(vtiles, utiles, d.B);
  if (accumulate)
    hipLaunchKernelGGL((pgrads_stream_kernel<true, false, TIO>), grid, dim3(256), 0, s, E, P, mE,
                       mP, Wt, deltas, pgrads, inLen, labLen, d, Up, Tw, sp, split);
  else
    hipLaunchKernelGGL((pgrads_stream_kernel<false, false, TIO>), grid, dim3(256), 0, s, E, P, mE,
                       mP, Wt, deltas, pgrads, inLen, labLen, d, Up, Tw, sp, split);
  RNNT_LAUNCH_CHECK("pgrads_stream_kernel");
  return kOk;
}
#if RNNT_IN_PART(3)
int launch_pgrads_stream(const float* E, const float* P, const float* mE, const float* mP,
                         const float* Wt, const float* deltas, float* pgrads, const int* inLen,
                         const int* labLen, const Dims& d, bool accumulate,
                         const SparsePTerms& sp, void* split_ws,
                         hipStream_t s) {
  return pgrads_stream_any(E, P, mE, mP, Wt, deltas, pgrads, inLen, labLen, d, accumulate, sp,
                           split_ws, s);
}
#endif
#if RNNT_IN_PART(4)
int launch_pgrads_stream(const bf16_t* E, const bf16_t* P, const float* mE, const float* mP,
                         const float* Wt, const float* deltas, bf16_t* pgrads, const int* inLen,
                         const int* labLen, const Dims& d, bool accumulate,
                         const SparsePTerms& sp, void* split_ws,
                         hipStream_t s) {
  return pgrads_stream_any(E, P, mE, mP, Wt, deltas, pgrads, inLen, labLen, d, accumulate, sp,
                           split_ws, s);
}
#endif
#if RNNT_IN_PART(5)
int launch_pgrads_stream(const f16_t* E, const f16_t* P, const float* mE, const float* mP,
                         const float* Wt, const float* deltas, f16_t* pgrads, const int* inLen,
                         const int* labLen, const Dims& d, bool accumulate,
                         const SparsePTerms& sp, void* split_ws,
                         hipStream_t s) {
  return pgrads_stream_any(E, P, mE, mP, Wt, deltas, pgrads, inLen, labLen, d, accumulate, sp,
                           split_ws, s);
}
#endif

}  // namespace rnnt
