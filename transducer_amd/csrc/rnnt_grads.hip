// Streaming forms of the two dense-gradient contractions (transducer/torch_binding.py:85-89)
// for gfx950.  Both keep the vocabulary-side operand of v_mfma_f32_32x32x2_f32 in REGISTERS,
// read straight from global memory in the instruction's own lane order (32 consecutive v per
// half-wave = one 128-byte line), and pass only the small W operand through LDS:
//
//   egrads[t,v] = delta * exp(E[t,v]-mE[t]) * sum_u Wn[t,u] * Y[u,v]      Y = exp(P-mP)
//       a wavefront owns 64 columns v and holds Y[:, its columns] (all label positions) in
//       registers for its whole life; it walks the frames 32 at a time, reads the 32 x U slab
//       of W from LDS, and multiplies the finished 32x64 block with exp(E-mE) on its way out.
//       E is read once and egrads written once, each as whole cache lines.
//
//   pgrads[u,v] = delta * exp(P[u,v]-mP[u]) * sum_t Wt[u,t] * X[t,v]      X = exp(E-mE)
//       a wavefront owns 32 columns v and all (up to 128) label positions; it walks the frames
//       32 at a time, turning the 32 x 32 slab of E it just loaded into X in registers.
//
// Which reduction element sits in which k-slot of the instruction is free as long as both
// operands agree: a lane takes four consecutive k of its W row with one 16-byte LDS read
// (k = 8j + 4*(lane/32) + q) and pairs them with the four matching register values.
#include "rnnt_internal.h"

namespace rnnt {

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
constexpr float kNegInf = -__builtin_huge_valf();

__device__ inline float f4at(const float4& v, int q) {
  return q == 0 ? v.x : (q == 1 ? v.y : (q == 2 ? v.z : v.w));
}

// ------------------------------------------------------------------ egrads
constexpr int kEsMaxG = 14;              // groups of 8 label positions kept in registers
constexpr int kEsKP = 8 * kEsMaxG + 4;   // LDS row pitch of the W slab (floats)

__global__ __launch_bounds__(256, 2) void egrads_stream_kernel(
    const float* __restrict__ E, const float* __restrict__ P, const float* __restrict__ mE,
    const float* __restrict__ mP, const float* __restrict__ Wn, const float* __restrict__ deltas,
    float* __restrict__ egrads, const int* __restrict__ inLen, const int* __restrict__ labLen,
    Dims d, int Up, int Tw, int tiles_per_chunk, int accumulate) {
  __shared__ __attribute__((aligned(16))) float As[2][32 * kEsKP];
  const int b = blockIdx.z;
  int Tb, Ub;
  utt_extent(inLen, labLen, b, d.T, d.U, Tb, Ub);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, h = lane >> 5;
  const int vcol = blockIdx.x * 256 + wave * 64 + l32;  // column of N-block 0; block 1 is +32
  const int ntiles = (d.T + 31) >> 5;
  const int tile_lo = blockIdx.y * tiles_per_chunk;
  const int tile_hi = min(tile_lo + tiles_per_chunk, ntiles);
  const int tile_valid = min(tile_hi, (Tb + 31) >> 5);  // tiles that hold frames of the utterance
  const int ngroups = (Ub + 7) >> 3;
  const float delta = deltas ? deltas[b] : 1.0f;
  const float* Eb = E + (size_t)b * d.T * d.V;
  float* out = egrads + (size_t)b * d.T * d.V;
  const float* mEb = mE + (size_t)b * d.T;
  const bool vok0 = vcol < d.V, vok1 = vcol + 32 < d.V;

  // Y fragments for this wavefront's 64 columns
  float Yr[kEsMaxG][4][2];
  {
    const float* Pb = P + (size_t)b * d.U * d.V;
    const float* mPb = mP + (size_t)b * d.U;
#pragma unroll
    for (int j = 0; j < kEsMaxG; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int u = 8 * j + 4 * h + q;
        float y0 = 0.0f, y1 = 0.0f;
        if (j < ngroups && u < Ub) {
          const float m = mPb[u];
          if (vok0) y0 = __expf(Pb[(size_t)u * d.V + vcol] - m);
          if (vok1) y1 = __expf(Pb[(size_t)u * d.V + vcol + 32] - m);
        }
        Yr[j][q][0] = y0;
        Yr[j][q][1] = y1;
      }
  }

  // W slab staging: the 32 x Up slab of frame tile ti is one contiguous run of 8*Up float4
  const int up4 = Up >> 2, nvec = 8 * Up;
  int lds_off[4];
  bool vec_ok[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int idx = tid + 256 * i;
    vec_ok[i] = idx < nvec;
    lds_off[i] = (idx / up4) * kEsKP + 4 * (idx % up4);
  }
  float4 areg[4];
  auto fetch_slab = [&](int ti) {
    const float4* src =
        reinterpret_cast<const float4*>(Wn + ((size_t)b * Tw + (size_t)ti * 32) * Up);
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (vec_ok[i]) areg[i] = src[tid + 256 * i];
  };
  auto store_slab = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (vec_ok[i]) *reinterpret_cast<float4*>(&As[buf][lds_off[i]]) = areg[i];
  };

  int cur = 0;
  if (tile_lo < tile_valid) {
    fetch_slab(tile_lo);
    store_slab(0);
  }
  __syncthreads();

  for (int ti = tile_lo; ti < tile_valid; ++ti) {
    const int t0 = ti * 32;
    const bool has_next = ti + 1 < tile_valid;
    if (has_next) fetch_slab(ti + 1);
    // the emissions of this tile, requested before the matrix work so they arrive under it
    float ev[16][2], mv[16];
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int t = t0 + 8 * (r >> 2) + 4 * h + (r & 3);
      const bool tok = t < Tb;
      const size_t o = (size_t)(tok ? t : 0) * d.V;
      mv[r] = mEb[tok ? t : 0];
      ev[r][0] = (tok && vok0) ? Eb[o + vcol] : kNegInf;
      ev[r][1] = (tok && vok1) ? Eb[o + vcol + 32] : kNegInf;
    }
    floatx16 acc0, acc1;
#pragma unroll
    for (int r = 0; r < 16; ++r) { acc0[r] = 0.0f; acc1[r] = 0.0f; }
#pragma unroll
    for (int j = 0; j < kEsMaxG; ++j) {
      if (j < ngroups) {
        const float4 a4 =
            *reinterpret_cast<const float4*>(&As[cur][l32 * kEsKP + 8 * j + 4 * h]);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float a = f4at(a4, q);
          acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, Yr[j][q][0], acc0, 0, 0, 0);
          acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a, Yr[j][q][1], acc1, 0, 0, 0);
        }
      }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int t = t0 + 8 * (r >> 2) + 4 * h + (r & 3);
      if (t < d.T) {
        const size_t o = (size_t)t * d.V + vcol;
        float g0 = __expf(ev[r][0] - mv[r]) * acc0[r];  // exp(-inf) = 0 on padded frames
        float g1 = __expf(ev[r][1] - mv[r]) * acc1[r];
        if (t >= Tb) { g0 = 0.0f; g1 = 0.0f; }
        if (vok0) out[o] = delta * (accumulate ? out[o] + g0 : g0);
        if (vok1) out[o + 32] = delta * (accumulate ? out[o + 32] + g1 : g1);
      }
    }
    if (has_next) store_slab(cur ^ 1);
    __syncthreads();
    cur ^= 1;
  }

  // frames past the utterance: the dense part is exactly zero
  for (int ti = max(tile_lo, tile_valid); ti < tile_hi; ++ti) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int t = ti * 32 + 8 * (r >> 2) + 4 * h + (r & 3);
      if (t < d.T) {
        const size_t o = (size_t)t * d.V + vcol;
        if (vok0) out[o] = accumulate ? delta * out[o] : 0.0f;
        if (vok1) out[o + 32] = accumulate ? delta * out[o + 32] : 0.0f;
      }
    }
  }
}

// ------------------------------------------------------------------ pgrads
constexpr int kPsKP = 32 + 4;  // LDS row pitch of the W^T slab (floats)

__global__ __launch_bounds__(256, 2) void pgrads_stream_kernel(
    const float* __restrict__ E, const float* __restrict__ P, const float* __restrict__ mE,
    const float* __restrict__ mP, const float* __restrict__ Wt, const float* __restrict__ deltas,
    float* __restrict__ pgrads, const int* __restrict__ inLen, const int* __restrict__ labLen,
    Dims d, int Up, int Tw, int accumulate) {
  __shared__ __attribute__((aligned(16))) float As[2][128 * kPsKP];
  const int b = blockIdx.z, u0 = blockIdx.y * 128;
  int Tb, Ub;
  utt_extent(inLen, labLen, b, d.T, d.U, Tb, Ub);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l32 = lane & 31, h = lane >> 5;
  const int vcol = blockIdx.x * 128 + wave * 32 + l32;
  const bool vok = vcol < d.V;
  const float delta = deltas ? deltas[b] : 1.0f;
  float* out = pgrads + (size_t)b * d.U * d.V;
  const int nmb = (u0 < Ub && Tb > 0) ? min(4, (Ub - u0 + 31) >> 5) : 0;  // 32-row blocks in use

  floatx16 acc[4];
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[mb][r] = 0.0f;

  if (nmb > 0) {
    const float* Eb = E + (size_t)b * d.T * d.V;
    const float* mEb = mE + (size_t)b * d.T;
    // W^T slab staging: 128 rows (u) x 32 frames = 1024 float4, four per thread
    const int arow = tid >> 3, ac4 = tid & 7;  // rows arow + 32*i
    float4 areg[4];
    auto fetch_slab = [&](int k0) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int u = u0 + arow + 32 * i;
        areg[i] = (i < nmb && u < Up)
                      ? *reinterpret_cast<const float4*>(Wt + ((size_t)b * Up + u) * Tw + k0 + 4 * ac4)
                      : make_float4(0.f, 0.f, 0.f, 0.f);
      }
    };
    auto store_slab = [&](int buf) {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        *reinterpret_cast<float4*>(&As[buf][(arow + 32 * i) * kPsKP + 4 * ac4]) = areg[i];
    };
    float xraw[4][4], xm[4][4];
    auto fetch_x = [&](int k0) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int t = k0 + 8 * j + 4 * h + q;
          const bool tok = t < Tb;
          xm[j][q] = mEb[tok ? t : 0];
          xraw[j][q] = (tok && vok) ? Eb[(size_t)t * d.V + vcol] : kNegInf;
        }
    };

    const int nk = (Tb + 31) >> 5;
    fetch_slab(0);
    fetch_x(0);
    store_slab(0);
    __syncthreads();
    int cur = 0;
    for (int kt = 0; kt < nk; ++kt) {
      float x[4][4];
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) x[j][q] = __expf(xraw[j][q] - xm[j][q]);
      const bool has_next = kt + 1 < nk;
      if (has_next) {
        fetch_slab((kt + 1) * 32);
        fetch_x((kt + 1) * 32);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) {
          if (mb < nmb) {
            const float4 a4 = *reinterpret_cast<const float4*>(
                &As[cur][(32 * mb + l32) * kPsKP + 8 * j + 4 * h]);
#pragma unroll
            for (int q = 0; q < 4; ++q)
              acc[mb] = __builtin_amdgcn_mfma_f32_32x32x2f32(f4at(a4, q), x[j][q], acc[mb], 0, 0, 0);
          }
        }
      if (has_next) store_slab(cur ^ 1);
      __syncthreads();
      cur ^= 1;
    }
  }

  const float* Pb = P + (size_t)b * d.U * d.V;
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int u = u0 + 32 * mb + 8 * (r >> 2) + 4 * h + (r & 3);
      if (u < d.U && vok) {
        const size_t o = (size_t)u * d.V + vcol;
        float g = 0.0f;
        if (mb < nmb && u < Ub) g = __expf(Pb[o] - mP[(size_t)b * d.U + u]) * acc[mb][r];
        out[o] = delta * (accumulate ? out[o] + g : g);
      }
    }
}

}  // namespace

#define RNNT_LAUNCH_CHECK(name)                                                    \
  do {                                                                             \
    hipError_t _e = hipGetLastError();                                             \
    if (_e != hipSuccess) return check_hip(_e, "launch " name, __FILE__, __LINE__); \
  } while (0)

bool egrads_stream_supported(const Dims& d) { return wplane_up(d.U) <= 8 * kEsMaxG; }

int launch_egrads_stream(const float* E, const float* P, const float* mE, const float* mP,
                         const float* Wn, const float* deltas, float* egrads, const int* inLen,
                         const int* labLen, const Dims& d, bool accumulate, hipStream_t s) {
  const int Up = wplane_up(d.U), Tw = wplane_tw(d.T);
  const int vtiles = (d.V + 255) / 256, ntiles = (d.T + 31) / 32;
  // enough workgroups to fill 256 CUs two deep several times over, but long enough runs of
  // frames per workgroup to amortise loading the Y fragments
  int chunks = (2048 + vtiles * d.B - 1) / (vtiles * d.B);
  chunks = chunks < 1 ? 1 : chunks;
  const int max_chunks = (ntiles + 7) / 8;
  if (chunks > max_chunks) chunks = max_chunks;
  const int per = (ntiles + chunks - 1) / chunks;
  chunks = (ntiles + per - 1) / per;
  hipLaunchKernelGGL(egrads_stream_kernel, dim3(vtiles, chunks, d.B), dim3(256), 0, s, E, P, mE,
                     mP, Wn, deltas, egrads, inLen, labLen, d, Up, Tw, per, accumulate ? 1 : 0);
  RNNT_LAUNCH_CHECK("egrads_stream_kernel");
  return kOk;
}

int launch_pgrads_stream(const float* E, const float* P, const float* mE, const float* mP,
                         const float* Wt, const float* deltas, float* pgrads, const int* inLen,
                         const int* labLen, const Dims& d, bool accumulate, hipStream_t s) {
  const int Up = wplane_up(d.U), Tw = wplane_tw(d.T);
  hipLaunchKernelGGL(pgrads_stream_kernel, dim3((d.V + 127) / 128, (d.U + 127) / 128, d.B),
                     dim3(256), 0, s, E, P, mE, mP, Wt, deltas, pgrads, inLen, labLen, d, Up, Tw,
                     accumulate ? 1 : 0);
  RNNT_LAUNCH_CHECK("pgrads_stream_kernel");
  return kOk;
}

}  // namespace rnnt
