// Row maxima of the score arrays, the W planes that feed the two gradient contractions, and
// the launchers of those contractions (rnnt_grads.hip).  W[t,u] = dalpha[t,u] / sum_v(...) as in
// the dense gradient parts of transducer/torch_binding.py:85-89:
//       egrads[t,v] = delta * exp(E[t,v]-mE[t]) * sum_u W[t,u] * exp(P[u,v]-mP[u])
//       pgrads[u,v] = delta * exp(P[u,v]-mP[u]) * sum_t W[t,u] * exp(E[t,v]-mE[t])
#include <type_traits>

#include "rnnt_internal.h"

namespace rnnt {

namespace {

constexpr float kNegInf = -__builtin_huge_valf();

__device__ inline float wave_max(float m) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
  return m;
}

// ------------------------------------------------------------------ row maxima
// 16-bit rows (V % 8 == 0 and 16-byte aligned when vec is set): eight elements per aligned load.
template <typename T16, typename = std::enable_if_t<sizeof(T16) == 2>>
__device__ inline float row_max(const T16* __restrict__ x, int V, int vec, int lane) {
  float m0 = kNegInf, m1 = kNegInf;
  if (vec) {
    for (int i = lane; i < (V >> 3); i += 64) {
      float e[8];
      expand(load8(x, 8 * i, V), e);
      m0 = fmaxf(m0, fmaxf(fmaxf(e[0], e[1]), fmaxf(e[2], e[3])));
      m1 = fmaxf(m1, fmaxf(fmaxf(e[4], e[5]), fmaxf(e[6], e[7])));
    }
  } else {
    // whole eights at the element type's own alignment, then the row's last few one by one
    for (int i = lane; i < (V >> 3); i += 64) {
      float e[8];
      expand(load8_any(x, 8 * i, V), e);
      m0 = fmaxf(m0, fmaxf(fmaxf(e[0], e[1]), fmaxf(e[2], e[3])));
      m1 = fmaxf(m1, fmaxf(fmaxf(e[4], e[5]), fmaxf(e[6], e[7])));
    }
    for (int i = (V & ~7) + lane; i < V; i += 64) m0 = fmaxf(m0, ldf(x + i));
  }
  return wave_max(fmaxf(m0, m1));
}

// One wavefront per row of a [rows, V] array.
// rows_per_item / lengths (optional): row r belongs to item r / rows_per_item and is skipped
// (maximum reported as 0, nothing read) when its index inside the item is >= lengths[item] + extra.
// Maximum of one row, computed by one wavefront (every lane gets the result).
__device__ inline float row_max(const float* __restrict__ x, int V, int vec4, int lane) {
  float m0 = kNegInf, m1 = kNegInf, m2 = kNegInf, m3 = kNegInf;
  if (vec4) {
    const float4* x4 = reinterpret_cast<const float4*>(x);
    const int n4 = V >> 2;
    int i = lane;
    for (; i + 192 < n4; i += 256) {
      const float4 a = x4[i], b = x4[i + 64], c = x4[i + 128], e = x4[i + 192];
      m0 = fmaxf(m0, fmaxf(fmaxf(a.x, a.y), fmaxf(a.z, a.w)));
      m1 = fmaxf(m1, fmaxf(fmaxf(b.x, b.y), fmaxf(b.z, b.w)));
      m2 = fmaxf(m2, fmaxf(fmaxf(c.x, c.y), fmaxf(c.z, c.w)));
      m3 = fmaxf(m3, fmaxf(fmaxf(e.x, e.y), fmaxf(e.z, e.w)));
    }
    for (; i < n4; i += 64) {
      const float4 a = x4[i];
      m0 = fmaxf(m0, fmaxf(fmaxf(a.x, a.y), fmaxf(a.z, a.w)));
    }
  } else {
    // whole eights as 4-byte aligned wide loads, then the row's last few one by one
    for (int i = lane; i < (V >> 3); i += 64) {
      float e[8];
      expand(load8_any(x, 8 * i, V), e);
      m0 = fmaxf(m0, fmaxf(fmaxf(e[0], e[1]), fmaxf(e[2], e[3])));
      m1 = fmaxf(m1, fmaxf(fmaxf(e[4], e[5]), fmaxf(e[6], e[7])));
    }
    for (int i = (V & ~7) + lane; i < V; i += 64) m0 = fmaxf(m0, x[i]);
  }
  return wave_max(fmaxf(fmaxf(m0, m1), fmaxf(m2, m3)));
}

template <typename TIO>
__global__ __launch_bounds__(256) void rowmax_kernel(const TIO* __restrict__ X,
                                                     float* __restrict__ out, long rows, int V,
                                                     int vec4, int rows_per_item,
                                                     const int* __restrict__ lengths, int extra) {
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= rows) return;
  if (lengths) {
    const long item = row / rows_per_item;
    if (row - item * rows_per_item >= lengths[item] + extra) {
      if (lane == 0) out[row] = 0.0f;
      return;
    }
  }
  const float m = row_max(X + (size_t)row * V, V, vec4, lane);
  if (lane == 0) out[row] = m;
}

// Row maxima of the predictions plus the elements of each row that the lattice recursions need,
// P[u, blank] and P[u, label_u], written to the small per-position vectors.
template <typename TIO>
__global__ __launch_bounds__(256) void rowmax_pick_p_kernel(const TIO* __restrict__ P,
                                                            float* __restrict__ mP,
                                                            const int* __restrict__ labels,
                                                            const int* __restrict__ labLen,
                                                            Planes p, Dims d, int vec4) {
  const long row = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= (long)d.B * d.U) return;
  const int b = (int)(row / d.U), u = (int)(row - (long)b * d.U);
  const int Ub = min(max(labLen[b], 0) + 1, d.U);
  if (u >= Ub) {
    if (lane == 0) mP[row] = 0.0f;
    return;
  }
  const TIO* x = P + (size_t)row * d.V;
  const float m = row_max(x, d.V, vec4, lane);
  if (lane == 0) {
    mP[row] = m;
    const bool has_label = labels != nullptr && (u + 1 < Ub);
    p.pb[(size_t)b * d.Ua + u] = ldf(x + d.blank);
    p.pl[(size_t)b * d.Ua + u] = has_label ? ldf(x + label_at(labels, d, b, u)) : 0.0f;
  }
}

// ------------------------------------------------------------------ W planes
// W[t,u] = dalpha[t,u] / sum_v(...) = dalpha[t,u] * exp((mE[t] + mP[u]) - LN[t,u]), written
// twice: Wn[b][t][Up] (u contiguous, feeds the egrads contraction) and Wt[b][u][Tw]
// (t contiguous, feeds the pgrads contraction).  Cells outside the utterance are zero.
__global__ __launch_bounds__(256) void wplanes_kernel(const float* __restrict__ lngrads,
                                                      const float* __restrict__ LN,
                                                      const float* __restrict__ mE,
                                                      const float* __restrict__ mP,
                                                      float* __restrict__ Wn,
                                                      float* __restrict__ Wt,
                                                      const int* __restrict__ inLen,
                                                      const int* __restrict__ labLen, Dims d,
                                                      int Up, int Tw) {
  __shared__ float tile[64][65];
  const int b = blockIdx.z, t0 = blockIdx.x * 64, u0 = blockIdx.y * 64;
  int Tb, Ub;
  utt_extent(inLen, labLen, b, d.T, d.U, Tb, Ub);
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int t = t0 + ty + 4 * i, u = u0 + tx;
    float w = 0.0f;
    if (t < Tb && u < Ub) {
      const size_t o = ((size_t)b * d.T + t) * d.U + u;
      const float me = mE[(size_t)b * d.T + t];
      w = lngrads[o] * expf((me + mP[(size_t)b * d.U + u]) - LN[o]) * frame_exp_correction(me);
    }
    tile[ty + 4 * i][tx] = w;
    if (t < Tw && u < Up) Wn[((size_t)b * Tw + t) * Up + u] = w;
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int u = u0 + ty + 4 * i, t = t0 + tx;
    if (t < Tw && u < Up) Wt[((size_t)b * Up + u) * Tw + t] = tile[tx][ty + 4 * i];
  }
}

}  // namespace

template <typename TIO>
static int rowmax_any(const TIO* X, float* rowmax, long rows, int V, int rows_per_item,
                      const int* lengths, int extra, hipStream_t s) {
  if (rows == 0) return kOk;
  const int vec4 = (V % RowAlign<TIO>::kElems == 0) && ((reinterpret_cast<uintptr_t>(X) & 15) == 0);
  hipLaunchKernelGGL(rowmax_kernel<TIO>, dim3((unsigned)((rows + 3) / 4)), dim3(256), 0, s, X,
                     rowmax, rows, V, vec4, rows_per_item, lengths, extra);
  RNNT_LAUNCH_CHECK("rowmax_kernel");
  return kOk;
}
int launch_rowmax(const float* X, float* rowmax, long rows, int V, int rows_per_item,
                  const int* lengths, int extra, hipStream_t s) {
  return rowmax_any(X, rowmax, rows, V, rows_per_item, lengths, extra, s);
}
int launch_rowmax(const bf16_t* X, float* rowmax, long rows, int V, int rows_per_item,
                  const int* lengths, int extra, hipStream_t s) {
  return rowmax_any(X, rowmax, rows, V, rows_per_item, lengths, extra, s);
}
int launch_rowmax(const f16_t* X, float* rowmax, long rows, int V, int rows_per_item,
                  const int* lengths, int extra, hipStream_t s) {
  return rowmax_any(X, rowmax, rows, V, rows_per_item, lengths, extra, s);
}

template <typename TIO>
static int rowmax_pick_p_any(const TIO* P, float* mP, const int* labels, const int* labLen,
                             const Planes& p, const Dims& d, hipStream_t s) {
  if (d.B == 0 || d.U == 0) return kOk;
  const int vp = (d.V % RowAlign<TIO>::kElems == 0) && ((reinterpret_cast<uintptr_t>(P) & 15) == 0);
  hipLaunchKernelGGL(rowmax_pick_p_kernel<TIO>, dim3((unsigned)(((long)d.B * d.U + 3) / 4)),
                     dim3(256), 0, s, P, mP, labels, labLen, p, d, vp);
  RNNT_LAUNCH_CHECK("rowmax_pick_p_kernel");
  return kOk;
}
int launch_rowmax_pick_p(const float* P, float* mP, const int* labels, const int* labLen,
                         const Planes& p, const Dims& d, hipStream_t s) {
  return rowmax_pick_p_any(P, mP, labels, labLen, p, d, s);
}
int launch_rowmax_pick_p(const bf16_t* P, float* mP, const int* labels, const int* labLen,
                         const Planes& p, const Dims& d, hipStream_t s) {
  return rowmax_pick_p_any(P, mP, labels, labLen, p, d, s);
}
int launch_rowmax_pick_p(const f16_t* P, float* mP, const int* labels, const int* labLen,
                         const Planes& p, const Dims& d, hipStream_t s) {
  return rowmax_pick_p_any(P, mP, labels, labLen, p, d, s);
}

int wplane_up(int U) { return (U + 7) & ~7; }
int wplane_tw(int T) { return (T + 63) & ~63; }

int launch_wplanes(const float* lngrads, const float* LN, const float* mE, const float* mP,
                   float* Wn, float* Wt, const int* inLen, const int* labLen, const Dims& d,
                   hipStream_t s) {
  if (d.B == 0 || d.T == 0 || d.U == 0) return kOk;
  const int Up = wplane_up(d.U), Tw = wplane_tw(d.T);
  hipLaunchKernelGGL(wplanes_kernel, dim3(Tw / 64, (Up + 63) / 64, d.B), dim3(256), 0, s, lngrads,
                     LN, mE, mP, Wn, Wt, inLen, labLen, d, Up, Tw);
  RNNT_LAUNCH_CHECK("wplanes_kernel");
  return kOk;
}

int launch_egrads(const float* E, const float* P, const float* mE, const float* mP,
                  const float* Wn, const float* deltas, float* egrads, const int* inLen,
                  const int* labLen, const Dims& d, bool accumulate, const SparseTerms& sparse,
                  hipStream_t s) {
  if (d.B == 0 || d.T == 0 || d.U == 0) return kOk;
  return launch_egrads_stream(E, P, mE, mP, Wn, deltas, egrads, inLen, labLen, d, accumulate,
                              sparse, s);
}

int launch_pgrads(const float* E, const float* P, const float* mE, const float* mP,
                  const float* Wt, const float* deltas, float* pgrads, const int* inLen,
                  const int* labLen, const Dims& d, bool accumulate, const SparsePTerms& sparse,
                  void* split_ws, hipStream_t s) {
  if (d.B == 0 || d.T == 0 || d.U == 0) return kOk;
  return launch_pgrads_stream(E, P, mE, mP, Wt, deltas, pgrads, inLen, labLen, d, accumulate,
                              sparse, split_ws, s);
}

}  // namespace rnnt
