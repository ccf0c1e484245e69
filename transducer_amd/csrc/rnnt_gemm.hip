// The three vocabulary-sized contractions of the RNN-T loss on the gfx950 matrix cores, with
// their exponentials and logarithms fused in so that nothing of size B*T*U*V -- and no copy of
// the [B,T,V] emissions -- ever goes to memory:
//
//   log-normaliser (transducer/torch_binding.py:35-40)
//       LN[t,u] = log( sum_v exp(E[t,v]-mE[t]) * exp(P[u,v]-mP[u]) ) + mE[t] + mP[u]
//   dense gradient parts (transducer/torch_binding.py:85-89), W[t,u] = dalpha[t,u]/sum_v(...)
//       egrads[t,v] = delta * exp(E[t,v]-mE[t]) * sum_u W[t,u] * exp(P[u,v]-mP[u])
//       pgrads[u,v] = delta * exp(P[u,v]-mP[u]) * sum_t W[t,u] * exp(E[t,v]-mE[t])
//
// All three use v_mfma_f32_32x32x2_f32 (fp32 in, fp32 accumulate).  A wavefront owns 32x32
// output blocks; for one instruction lane l supplies A[row l%32][k-slot l/32] and
// B[k-slot l/32][col l%32] and receives D[8*(r/4) + 4*(l/32) + r%4][l%32] in register r.
// Which element of the reduction sits in which k-slot is free as long as A and B agree, so a
// lane takes four consecutive k of its row with one 16-byte LDS read and spends them on four
// instructions.
#include <type_traits>

#include "rnnt_internal.h"

namespace rnnt {

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

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

// Row maxima of the emissions plus the elements of each row that the lattice recursions need:
// E[t, blank] and E[t, label_u] for every label position, written to the skewed planes (what
// gather_kernel of rnnt_dp.hip does with one scattered HBM sector per element; here the sectors
// are part of the row that is being streamed anyway).  A workgroup takes 16 consecutive frames of
// one utterance, four per wavefront; the picked scores meet in LDS and leave as runs of 16
// consecutive frames per label position.  Frames past the utterance are skipped.
constexpr int kPickRows = 16, kPickU = 256;

__global__ __launch_bounds__(256) void rowmax_pick_e_kernel(const float* __restrict__ E,
                                                            float* __restrict__ mE,
                                                            const int* __restrict__ labels,
                                                            const int* __restrict__ inLen,
                                                            const int* __restrict__ labLen,
                                                            Planes p, Dims d, int vec4) {
  __shared__ float tile[kPickRows][kPickU + 1];
  __shared__ float blanks[kPickRows];
  const int b = blockIdx.y, t0 = blockIdx.x * kPickRows;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int Tb, Ub;
  utt_extent(inLen, labLen, b, d.T, d.U, Tb, Ub);
  const int nlab = labels ? max(Ub - 1, 0) : 0;
  // label columns of this lane (first kPickU label positions)
  int col[kPickU / 64];
#pragma unroll
  for (int i = 0; i < kPickU / 64; ++i) {
    const int u = lane + 64 * i;
    col[i] = u < nlab ? labels[(size_t)b * (d.U - 1) + u] : d.blank;
  }
  // The picks of a frame are requested right after its row has been streamed (they hit L2) and
  // are put away after the NEXT row's stream, so their latency is never waited for.
  float pick[kPickU / 64], xb = 0.0f;
  int pending = -1;  // tile row the registers belong to
  auto put_away = [&]() {
    if (pending < 0) return;
#pragma unroll
    for (int k = 0; k < kPickU / 64; ++k) tile[pending][lane + 64 * k] = pick[k];
    if (lane == 0) blanks[pending] = xb;
    pending = -1;
  };
  for (int r = 0; r < 4; ++r) {
    const int i = 4 * wave + r, t = t0 + i;
    if (t >= d.T) break;
    const size_t row = (size_t)b * d.T + t;
    if (t >= Tb) {
      if (lane == 0) mE[row] = 0.0f;
      continue;
    }
    const float* x = E + row * d.V;
    const float m = row_max(x, d.V, vec4, lane);
    if (lane == 0) mE[row] = m;
    put_away();
#pragma unroll
    for (int k = 0; k < kPickU / 64; ++k) pick[k] = x[col[k]];
    xb = x[d.blank];
    pending = i;
    // label positions past the first kPickU: straight from the row
    for (int u = kPickU + lane; u < nlab; u += 64)
      p.elS[plane_row(d, b, u) + t + u] = x[labels[(size_t)b * (d.U - 1) + u]];
  }
  put_away();
  __syncthreads();
  const int nrows = min(kPickRows, Tb - t0);  // may be <= 0
  if ((int)threadIdx.x < nrows) p.eb[(size_t)b * d.Tp + d.Eo + t0 + threadIdx.x] = blanks[threadIdx.x];
  const int nu = min(nlab, kPickU);
  for (int idx = threadIdx.x; idx < nu * kPickRows; idx += 256) {
    const int u = idx >> 4, i = idx & 15;
    if (i < nrows) p.elS[plane_row(d, b, u) + t0 + i + u] = tile[i][u];
  }
}

// The same for the predictions: P[u, blank] and P[u, label_u].
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
    p.pl[(size_t)b * d.Ua + u] = has_label ? ldf(x + labels[(size_t)b * (d.U - 1) + u]) : 0.0f;
  }
}

// ------------------------------------------------------------------ log-normaliser, any shape
// Scalar-load form for vocabularies that are not a multiple of 4 or unaligned inputs.
// Block tile 128 (t) x 128 (u), reduction over v in slices of 32; 4 wavefronts, each 64x64.
// Both operands are v-contiguous in memory and are staged as S[row][v] with a 36-float pitch
// (16-byte reads of consecutive rows then fall into distinct bank groups).
constexpr int kLseBM = 128, kLseBN = 128, kLseBK = 32, kLsePitch = kLseBK + 4;

__global__ __launch_bounds__(256, 2) void lse_kernel(const float* __restrict__ E,
                                                     const float* __restrict__ P,
                                                     const float* __restrict__ mE,
                                                     const float* __restrict__ mP,
                                                     float* __restrict__ LN,
                                                     const int* __restrict__ inLen,
                                                     const int* __restrict__ labLen, Dims d) {
  __shared__ __attribute__((aligned(16))) float As[kLseBM * kLsePitch];
  __shared__ __attribute__((aligned(16))) float Bs[kLseBN * kLsePitch];
  const int b = blockIdx.z, t0 = blockIdx.x * kLseBM, u0 = blockIdx.y * kLseBN;
  int Tb, Ub;
  utt_extent(inLen, labLen, b, d.T, d.U, Tb, Ub);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  float* LNb = LN + (size_t)b * d.T * d.U;

  if (t0 >= Tb || u0 >= Ub) {
    // nothing valid here: the array still gets defined contents (zeros, as in the torch-free
    // reference helper transducer/test.h:58)
    for (int e = tid; e < kLseBM * kLseBN; e += 256) {
      const int t = t0 + e / kLseBN, u = u0 + e % kLseBN;
      if (t < d.T && u < d.U) LNb[(size_t)t * d.U + u] = 0.0f;
    }
    return;
  }

  const float* Eb = E + (size_t)b * d.T * d.V;
  const float* Pb = P + (size_t)b * d.U * d.V;
  const float* mEb = mE + (size_t)b * d.T;
  const float* mPb = mP + (size_t)b * d.U;

  // staging assignment: element e = tid + 256*i -> row e/32, column e%32 (a wavefront reads two
  // 128-byte row segments per load instruction)
  const int lcol = tid & 31, lrow0 = tid >> 5;  // rows lrow0 + 8*i, i < 16
  float ra[16], rb[16];
  float ma[16], mb[16];
  const float* pa[16];
  const float* pb[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int r = lrow0 + 8 * i;
    const int t = min(t0 + r, d.T - 1), u = min(u0 + r, d.U - 1);
    pa[i] = Eb + (size_t)t * d.V;
    pb[i] = Pb + (size_t)u * d.V;
    ma[i] = mEb[t];
    mb[i] = mPb[u];
  }
  auto fetch = [&](int k0) {
    const int v = k0 + lcol;
    const bool ok = v < d.V;
    const int vc = ok ? v : d.V - 1;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float x = pa[i][vc], y = pb[i][vc];
      ra[i] = ok ? x : kNegInf;  // exp(-inf - m) = 0: past-the-end terms add nothing
      rb[i] = ok ? y : kNegInf;
    }
  };

  const int wm = wave >> 1, wn = wave & 1, l32 = lane & 31, h = lane >> 5;
  floatx16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  const int nk = (d.V + kLseBK - 1) / kLseBK;
  fetch(0);
  for (int kt = 0; kt < nk; ++kt) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int r = lrow0 + 8 * i;
      As[r * kLsePitch + lcol] = __expf(ra[i] - ma[i]);
      Bs[r * kLsePitch + lcol] = __expf(rb[i] - mb[i]);
    }
    __syncthreads();
    if (kt + 1 < nk) fetch((kt + 1) * kLseBK);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float4 a4[2], b4[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        a4[i] = *reinterpret_cast<const float4*>(
            &As[(64 * wm + 32 * i + l32) * kLsePitch + 8 * j + 4 * h]);
        b4[i] = *reinterpret_cast<const float4*>(
            &Bs[(64 * wn + 32 * i + l32) * kLsePitch + 8 * j + 4 * h]);
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int jj = 0; jj < 2; ++jj) {
            const float av = q == 0 ? a4[i].x : (q == 1 ? a4[i].y : (q == 2 ? a4[i].z : a4[i].w));
            const float bv =
                q == 0 ? b4[jj].x : (q == 1 ? b4[jj].y : (q == 2 ? b4[jj].z : b4[jj].w));
            acc[i][jj] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc[i][jj], 0, 0, 0);
          }
      }
    }
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int jj = 0; jj < 2; ++jj)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int t = t0 + 64 * wm + 32 * i + 8 * (r >> 2) + 4 * h + (r & 3);
        const int u = u0 + 64 * wn + 32 * jj + l32;
        if (t < d.T && u < d.U) {
          float v = 0.0f;
          if (t < Tb && u < Ub) v = (logf(acc[i][jj][r]) + mEb[t]) + mPb[u];
          LNb[(size_t)t * d.U + u] = v;
        }
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
      w = lngrads[o] * expf((mE[(size_t)b * d.T + t] + mP[(size_t)b * d.U + u]) - LN[o]);
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

#define RNNT_LAUNCH_CHECK(name)                                                    \
  do {                                                                             \
    hipError_t _e = hipGetLastError();                                             \
    if (_e != hipSuccess) return check_hip(_e, "launch " name, __FILE__, __LINE__); \
  } while (0)

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

int launch_rowmax_pick(const float* E, const float* P, float* mE, float* mP, const int* labels,
                       const int* inLen, const int* labLen, const Planes& p, const Dims& d,
                       hipStream_t s) {
  if (d.B == 0 || d.T == 0 || d.U == 0) return kOk;
  const int ve = (d.V % 4 == 0) && ((reinterpret_cast<uintptr_t>(E) & 15) == 0);
  const int vp = (d.V % 4 == 0) && ((reinterpret_cast<uintptr_t>(P) & 15) == 0);
  hipLaunchKernelGGL(rowmax_pick_e_kernel, dim3((d.T + kPickRows - 1) / kPickRows, d.B), dim3(256),
                     0, s, E, mE, labels, inLen, labLen, p, d, ve);
  RNNT_LAUNCH_CHECK("rowmax_pick_e_kernel");
  hipLaunchKernelGGL(rowmax_pick_p_kernel<float>, dim3((unsigned)(((long)d.B * d.U + 3) / 4)),
                     dim3(256), 0, s, P, mP, labels, labLen, p, d, vp);
  RNNT_LAUNCH_CHECK("rowmax_pick_p_kernel");
  return kOk;
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

int launch_lse(const float* E, const float* P, const float* mE, const float* mP, float* LN,
               const int* inLen, const int* labLen, const Dims& d, hipStream_t s) {
  if (d.B == 0 || d.T == 0 || d.U == 0) return kOk;
  hipLaunchKernelGGL(lse_kernel,
                     dim3((d.T + kLseBM - 1) / kLseBM, (d.U + kLseBN - 1) / kLseBN, d.B),
                     dim3(256), 0, s, E, P, mE, mP, LN, inLen, labLen, d);
  RNNT_LAUNCH_CHECK("lse_kernel");
  return kOk;
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
