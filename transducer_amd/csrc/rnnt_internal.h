// Internal declarations shared by the HIP translation units of librnnt_hip.so.
// Nothing here is part of the public interface (see include/rnnt_hip.h for that).
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "rnnt_io.h"

namespace rnnt {

// ---------------------------------------------------------------- status / errors
enum Status { kOk = 0, kInvalid = 1, kHipError = 2, kWorkspace = 3 };

// Records a message for rnnt_hip_last_error() (thread-local) and returns `code`.
int fail(int code, const char* fmt, ...);
int check_hip(hipError_t e, const char* what, const char* file, int line);

#define RNNT_HIP(call)                                                   \
  do {                                                                   \
    int _st = ::rnnt::check_hip((call), #call, __FILE__, __LINE__);      \
    if (_st != ::rnnt::kOk) return _st;                                  \
  } while (0)

#define RNNT_TRY(expr)                 \
  do {                                 \
    int _st = (expr);                  \
    if (_st != ::rnnt::kOk) return _st; \
  } while (0)

// After a kernel launch inside a function that returns a status: the launch error, if any.
#define RNNT_LAUNCH_CHECK(name)                                                             \
  do {                                                                                      \
    hipError_t _e = hipGetLastError();                                                      \
    if (_e != hipSuccess) return ::rnnt::check_hip(_e, "launch " name, __FILE__, __LINE__); \
  } while (0)

// ---------------------------------------------------------------- geometry
// Problem sizes in the reference's vocabulary: U is the prediction length (longest label + 1).
struct Dims {
  int B, T, U, V, blank;
  int Ua;  // label positions per utterance in a skewed plane: U rounded up to 64 * cells-per-lane
  int Dp;  // anti-diagonals per utterance in a skewed plane (a multiple of four)
  int Tp;  // row pitch of the per-frame blank-score array
  int Eo;  // index of frame 0 inside a row of that array (frames -Eo..-1 are readable padding)
};

// A skewed plane stores cell (t,u) of utterance b by its anti-diagonal dd = t+u, four
// anti-diagonals to a group: [b][dd/4][u][dd%4].  All lanes of the wavefront that walks the lattice
// read the same anti-diagonals at the same step, so four consecutive steps are one aligned 16-byte
// load per lane, and the loads of neighbouring label positions are neighbours in memory: a load
// instruction of the walk touches 8 cache lines (one label position a lane), not 64 as with one
// row per label position (measured on the dalpha walk, B=32 T=2000 U=100: 71 -> 37 ns a step).
// Dp, the anti-diagonals a plane has room for (a multiple of four), leaves room for the last
// partial group of four and for the neighbours (t+1,u), (t,u+1) of the last cells.
__host__ __device__ inline int plane_pitch(int T, int U) { return ((T + U + 3) & ~3) + 8; }

// Label positions one lane would own if one wavefront took the whole label axis: a power of two.
// It sets the row count of the skewed planes (Ua = 64 x this); the walks themselves give a lane at
// most 16 positions and take a longer axis in blocks of 1024.
inline int cells_per_lane(int U) {
  int c = 1;
  while (c * 64 < U) c *= 2;
  return c;
}

inline Dims make_dims(int B, int T, int U, int V, int blank) {
  Dims d;
  d.B = B; d.T = T; d.U = U; d.V = V; d.blank = blank;
  d.Ua = 64 * cells_per_lane(U);
  d.Dp = plane_pitch(T, U);
  d.Eo = d.Ua + 4;
  d.Tp = d.Eo + ((T + U + 3) & ~3) + 8;
  return d;
}

// Offset of cell (u, anti-diagonal dd) of utterance b in a skewed plane.  Its neighbours: the same
// anti-diagonal of position u+1 is 4 floats further on; anti-diagonal dd+1 is plane_at(.., dd+1)
// (1 float further on inside a group of four, else in the next group).
__host__ __device__ inline size_t plane_at(const Dims& d, int b, int u, int dd) {
  return (size_t)b * d.Ua * d.Dp + ((size_t)(dd >> 2) * d.Ua + u) * 4 + (dd & 3);
}
// Offset of group 0 (anti-diagonals 0..3) of position u, and the distance between groups.
__host__ __device__ inline size_t plane_group0(const Dims& d, int b, int u) {
  return (size_t)b * d.Ua * d.Dp + 4 * (size_t)u;
}
__host__ __device__ inline int plane_group_stride(const Dims& d) { return 4 * d.Ua; }

__device__ inline int clampi(int x, int lo, int hi) { return x < lo ? lo : (x > hi ? hi : x); }

// Per-utterance extents, clamped to the padded array so a bad length can never index past it.
__device__ inline void utt_extent(const int* inLen, const int* labLen, int b, int T, int U,
                                  int& Tb, int& Ub) {
  Tb = inLen ? clampi(inLen[b], 0, T) : T;
  Ub = labLen ? clampi(labLen[b] + 1, 0, U) : U;
}

// Label of position u of utterance b, forced into the vocabulary.  The reference indexes its
// score rows with whatever the caller wrote (transducer/transducer_cpu.cpp:63-66); here every
// kernel reads labels through this one function, so a value outside [0, V) can neither read nor
// write past a row and all kernels agree on which column it means.
__device__ inline int label_at(const int* __restrict__ labels, const Dims& d, int b, int u) {
  return clampi(labels[(size_t)b * (d.U - 1) + u], 0, d.V - 1);
}

// Buffers of the lattice recursions, all in the skewed layout except the three small vectors.
struct Planes {
  float* lnS;   // log-normaliser LN[t,u]
  float* elS;   // E[t, label_u]  (label-move emission score of the cell)
  float* aS;    // alpha
  float* wB;    // blank-move weight exp(stay(t,u) - alpha[t+1,u])
  float* wE;    // label-move weight exp(emit(t,u) - alpha[t,u+1])
  float* dS;    // dalpha (= d cost / d LN)
  float* eb;    // E[t, blank] at [b*Tp + Eo + t]
  float* pb;    // P[u, blank]           [B, Ua]
  float* pl;    // P[u, label_u]         [B, Ua]
  float* gB;    // per-(b,u) blank-column sum of the sparse pgrads term   [B, Ua]
  float* gL;    // per-(b,u) label-column sum of the sparse pgrads term   [B, Ua]
  float* hand[2];  // [B, Dp] each: what crosses from one block of 1024 label positions to the
                   // next when a lattice walk takes the label axis block by block
};

// Trips a wavefront of the lattice kernels may spend waiting for its neighbour's progress
// counter before it gives up and raises the trouble flag (each trip is an LDS read and a short
// sleep, roughly 50 ns; the longest legitimate wait is a few dozen trips).
constexpr int kDefaultSpinLimit = 1 << 20;
extern int g_spin_limit;
// Device address of the current device's trouble flag (a static device int, looked up once per
// device).
int trouble_flag(int** out);

// One wavefront running `steps` steps of the bare dependent chain of an alpha (kind 0) or dalpha
// (kind 1) cell; see chain_floor_kernel.
int launch_chain_floor(int kind, int steps, hipStream_t s);
// expf_glibc / log1pf_glibc (rnnt_libm.h) of n floats, for the tests.
int launch_libm_probe(const float* x, float* e, float* l, long n, hipStream_t s);
// out[0] += number of floats d <= 0 with bit pattern in [lo, hi] for which the error bound of the
// fast log-sum-exp fails, out[1] = max(out[1], bits of the largest distance / bound).
int launch_lse_bound_check(unsigned lo, unsigned hi, unsigned* out, hipStream_t s);

// decode_only: just what the best-path walk reads (the LN plane and the small vectors); the
// five other lattice planes are left out and their pointers null.
size_t planes_bytes(const Dims& d, bool decode_only = false);
void carve_planes(void* base, const Dims& d, Planes* p, bool decode_only = false);

// ---------------------------------------------------------------- launchers (rnnt_dp.hip)
int launch_skew(const float* src, float* dstS, const int* inLen, const int* labLen, const Dims& d,
                hipStream_t s);
int launch_unskew(const float* srcS, float* dst, const int* inLen, const int* labLen,
                  const Dims& d, hipStream_t s);
int launch_gather(const float* E, const float* P, const int* labels, const int* inLen,
                  const int* labLen, const Planes& p, const Dims& d, hipStream_t s);
int launch_gather(const bf16_t* E, const bf16_t* P, const int* labels, const int* inLen,
                  const int* labLen, const Planes& p, const Dims& d, hipStream_t s);
int launch_gather(const f16_t* E, const f16_t* P, const int* labels, const int* inLen,
                  const int* labLen, const Planes& p, const Dims& d, hipStream_t s);
int launch_alpha(const Planes& p, const int* inLen, const int* labLen, float* costs,
                 const Dims& d, hipStream_t s);
int launch_weights(const Planes& p, const int* inLen, const int* labLen, const Dims& d,
                   hipStream_t s);
int launch_beta(const Planes& p, const int* labels, const int* inLen, const int* labLen,
                const Dims& d, hipStream_t s);
// Sparse blank/label terms.  add == false: written onto zero-filled egrads/pgrads exactly as
// the reference's backward leaves them.  add == true: added, times scale[b] (1 when scale is
// null), onto arrays that already hold the dense part.
// pgrads == nullptr: only the egrads terms.  bsum ([B,T]) and emT ([B,U,T]) are the per-frame
// terms launch_post_beta forms from the finished dalpha plane.
int launch_sparse(const Planes& p, const float* bsum, const float* emT, float* egrads,
                  float* pgrads, const int* labels, const int* inLen, const int* labLen,
                  const float* scale, bool add, const Dims& d, hipStream_t s);
// After the dalpha walk, in one launch: the W planes (both orientations, from the skewed dalpha
// and LN planes) and, with bsum != nullptr, bsum[b,t] = what the blank/label terms leave in
// egrads[b,t,blank] (for folding into the dense kernel's write-out).
// With `img` set, W is left as bf16 pieces in the slab images of the fused gradient kernel
// instead of the two fp32 planes (Wn, Wt are then not written).
struct WImages {
  // One image per (utterance, slab of 32 frames), three planes (the bf16 pieces, largest first):
  //   e: [32 frames][kCols label positions]          -- the A operand of the egrads products
  //   p: [128 label positions][32 frame slots]       -- the A operand of the pgrads products,
  //      the frames of a slab in the order the fused kernel's matrix instructions take them
  // as 32-bit words of two bf16 each.  Zero outside the utterance.
  static constexpr int kCols = 112;
  static constexpr int kEPlane = 32 * kCols / 2;  // words per plane
  static constexpr int kPPlane = 128 * 32 / 2;
  unsigned* e = nullptr;
  unsigned* p = nullptr;
  static size_t e_bytes(int B, int Tw) { return (size_t)B * (Tw / 32) * 3 * kEPlane * 4; }
  static size_t p_bytes(int B, int Tw) { return (size_t)B * (Tw / 32) * 3 * kPPlane * 4; }
};
// bsum ([B,T]) and emT ([B,U,T]): the per-frame blank totals and the per-cell label-move terms
// that the dense egrads kernel folds in (SparseTerms) or launch_sparse scatters; both null: not
// formed.  Wn == nullptr (and no images): no W planes, only those terms (mE, mP unused).
int launch_post_beta(const Planes& p, const float* mE, const float* mP, float* Wn, float* Wt,
                     float* bsum, float* emT, const int* labels, const int* inLen,
                     const int* labLen, const Dims& d, hipStream_t s,
                     const WImages& img = WImages());
// best / arg: skewed planes (see plane_at), written for valid cells only.
int launch_maxplus(const float* E, const float* P, const int* inLen, const int* labLen,
                   float* best, int* arg, const Dims& d, hipStream_t s, void* lists = nullptr,
                   bool force = false);
int launch_maxplus(const bf16_t* E, const bf16_t* P, const int* inLen, const int* labLen,
                   float* best, int* arg, const Dims& d, hipStream_t s, void* lists = nullptr,
                   bool force = false);
int launch_maxplus(const f16_t* E, const f16_t* P, const int* inLen, const int* labLen,
                   float* best, int* arg, const Dims& d, hipStream_t s, void* lists = nullptr,
                   bool force = false);
// `lists`: maxplus_lists_bytes(d) bytes of scratch, or null (plan 0); force: plan 2.  With it, and where
// maxplus_plan(d) says so, most cells are settled from short candidate lists
// (rnnt_cand.hip) and only the cells whose bound test fails are evaluated over every column.
bool maxplus_lists_possible(const Dims& d);
bool maxplus_lists_pay(const Dims& d);
// How a call of this shape builds its table under the current mode, decided ONCE per call (the
// mode is process-wide and another thread may change it): 0 over every column, 1 from lists if
// the sample of cells agrees, 2 from lists unconditionally.
int maxplus_plan(const Dims& d);
size_t maxplus_lists_bytes(const Dims& d);
void set_maxplus_mode(int mode);
int maxplus_tile_limit();
void maxplus_lists_counters(void* scratch, const Dims& d, const int** tile_fail,
                            const int** lists_on);
#define RNNT_DECLARE_LISTS(T)                                                                   \
  int launch_maxplus_lists(const T* E, const T* P, const int* inLen, const int* labLen,        \
                           float* best, int* arg, const Dims& d, void* scratch, bool force,       \
                           hipStream_t s);                                                      \
  int launch_maxplus_cells(const T* E, const T* P, const int* inLen, const int* labLen,        \
                           float* best, int* arg, const Dims& d, void* scratch, hipStream_t s);
RNNT_DECLARE_LISTS(float)
RNNT_DECLARE_LISTS(bf16_t)
RNNT_DECLARE_LISTS(f16_t)
#undef RNNT_DECLARE_LISTS
int launch_table_out(const float* bestS, const int* argS, const int* inLen, const int* labLen,
                     float* best, int* arg, const Dims& d, hipStream_t s);
// bestS / argS: skewed planes of the max-plus table (argS carries int bits in float storage).
int launch_viterbi(const Planes& p, const float* bestS, const float* argS,
                   unsigned long long* gbits, const int* inLen, const int* labLen,
                   int* labels_out, const Dims& d, hipStream_t s);
size_t viterbi_bits_bytes(const Dims& d);

// ---------------------------------------------------------------- launchers (rnnt_prep.hip)
// The gradient kernels form exp(E[t,v] - mE[t]) as exp2(fma(E, log2 e, -fl(mE log2 e))): one
// fused multiply-add and one v_exp_f32 per element.  The rounding of the product mE log2 e makes
// every exponential of frame t too large by the same factor 2^r, r = mE log2 e - fl(mE log2 e)
// (up to 2^-24 |mE log2 e|: 2e-7 at |mE| = 4, but 6e-6 at 100 and past the gradients' tolerance
// from |mE| of about 1700).  Both gradients are linear in W[t,u] x exp(E[t,v] - mE[t]), so the
// kernels that write W multiply it by 2^-r of its frame and the hot loops stay as they are.
constexpr float kLog2eF = 1.44269504088896340736f;
__device__ inline float frame_exp_correction(float mE) {
  const float hi = mE * kLog2eF;  // (rounded: what the gradient kernels subtract)
  const float r = __builtin_fmaf(mE, kLog2eF, -hi);
  return __builtin_amdgcn_exp2f(-r);
}
int wplane_up(int U);  // label-axis pitch of the W planes (multiple of 8)
int wplane_tw(int T);  // frame-axis pitch of the W planes (multiple of 64)
// Row maxima of a [rows, V] array.  With `lengths`, rows at or past lengths[item] + extra inside
// their item (rows_per_item rows each) are not read and report 0.
int launch_rowmax(const float* X, float* rowmax, long rows, int V, int rows_per_item,
                  const int* lengths, int extra, hipStream_t s);
int launch_rowmax(const bf16_t* X, float* rowmax, long rows, int V, int rows_per_item,
                  const int* lengths, int extra, hipStream_t s);
int launch_rowmax(const f16_t* X, float* rowmax, long rows, int V, int rows_per_item,
                  const int* lengths, int extra, hipStream_t s);
// Log-normaliser (rnnt_lse.hip): any V; 16-byte row loads when V is a multiple of
// the vector width and E is 16-byte aligned, element loads otherwise.  The pieces of
// exp(P - mP) are first written to `scratch` (lse_scratch_bytes) in matrix-operand order.
// launch_lse_stream needs mP only and WRITES mE (one reference value per frame, >= the row
// maximum minus a fixed slack; what the gradient kernels need as mE).
// Each launcher that reads the scores or writes their gradients exists for fp32, bf16 and
// fp16 arrays (rnnt_io.h).
bool lse_stream_supported(const float* E, const Dims& d);
bool lse_stream_supported(const bf16_t* E, const Dims& d);
bool lse_stream_supported(const f16_t* E, const Dims& d);
size_t lse_scratch_bytes(const Dims& d);
int launch_yplanes(const float* P, const float* mP, void* scratch, const int* labLen,
                   const Dims& d, hipStream_t s);
int launch_yplanes(const bf16_t* P, const float* mP, void* scratch, const int* labLen,
                   const Dims& d, hipStream_t s);
int launch_yplanes(const f16_t* P, const float* mP, void* scratch, const int* labLen,
                   const Dims& d, hipStream_t s);
// With elS / eb (skewed label-score plane and blank-score vector) it also copies E[t, label_u]
// and E[t, blank] out of the rows it streams (what launch_gather does for the emissions).
// With lnS it writes LN into that skewed plane (valid cells) INSTEAD of the row-major LN.
int launch_lse_stream(const float* E, float* mE, const float* mP, float* LN,
                      const void* scratch, const int* inLen, const int* labLen, const Dims& d,
                      hipStream_t s, const int* labels = nullptr, float* elS = nullptr,
                      float* eb = nullptr, float* lnS = nullptr);
int launch_lse_stream(const bf16_t* E, float* mE, const float* mP, float* LN,
                      const void* scratch, const int* inLen, const int* labLen, const Dims& d,
                      hipStream_t s, const int* labels = nullptr, float* elS = nullptr,
                      float* eb = nullptr, float* lnS = nullptr);
int launch_lse_stream(const f16_t* E, float* mE, const float* mP, float* LN,
                      const void* scratch, const int* inLen, const int* labLen, const Dims& d,
                      hipStream_t s, const int* labels = nullptr, float* elS = nullptr,
                      float* eb = nullptr, float* lnS = nullptr);
// P[u, blank] and P[u, label_u] into the planes, with the row maxima of P (one pass).
int launch_rowmax_pick_p(const float* P, float* mP, const int* labels, const int* labLen,
                         const Planes& p, const Dims& d, hipStream_t s);
int launch_rowmax_pick_p(const bf16_t* P, float* mP, const int* labels, const int* labLen,
                         const Planes& p, const Dims& d, hipStream_t s);
int launch_rowmax_pick_p(const f16_t* P, float* mP, const int* labels, const int* labLen,
                         const Planes& p, const Dims& d, hipStream_t s);
int launch_wplanes(const float* lngrads, const float* LN, const float* mE, const float* mP,
                   float* Wn, float* Wt, const int* inLen, const int* labLen, const Dims& d,
                   hipStream_t s);
// Sparse blank/label terms of egrads for folding into the dense kernel's write-out: with
// labels != nullptr, out = delta * (dense + sparse) (needs accumulate == false).
struct SparseTerms {
  const float* emT = nullptr;   // [B,U,T] label-move terms dalpha[t,u+1] wE[t,u]
  const float* bsum = nullptr;  // [B,T] blank-column totals
  const int* labels = nullptr;  // [B,U-1]
};
// The same for pgrads: per-(b,u) totals of the blank and the label column (Planes::gB, gL), added
// in the dense kernel's write-out exactly as sparse_p_kernel would add them afterwards.
struct SparsePTerms {
  const float* gB = nullptr;
  const float* gL = nullptr;
  const int* labels = nullptr;  // [B,U-1]; may be null when U == 1
};
// accumulate == false: out = delta * dense.   accumulate == true: out = delta * (out + dense),
// the update of transducer/torch_binding.py:86-89.
int launch_egrads(const float* E, const float* P, const float* mE, const float* mP,
                  const float* Wn, const float* deltas, float* egrads, const int* inLen,
                  const int* labLen, const Dims& d, bool accumulate, const SparseTerms& sparse,
                  hipStream_t s);
// split_ws: pgrads_split_bytes(d) bytes of scratch that let several workgroups share a tile's
// frames when the grid is small (null: one workgroup per tile).
size_t pgrads_split_bytes(const Dims& d);
int launch_pgrads(const float* E, const float* P, const float* mE, const float* mP,
                  const float* Wt, const float* deltas, float* pgrads, const int* inLen,
                  const int* labLen, const Dims& d, bool accumulate, const SparsePTerms& sparse,
                  void* split_ws, hipStream_t s);


// ---------------------------------------------------------------- launchers (rnnt_grads.hip)
// Both dense gradients from one walk over the frames (each row of E read once); needs the
// blank / label terms folded into both write-outs.
bool grads_fused_possible(const Dims& d);  // the kernel can take this shape
bool grads_fused_pays(const Dims& d);      // ... and is expected to beat the two contractions
int launch_grads_fused(const float* E, const float* P, const float* mE, const float* mP,
                       const WImages& img, const float* deltas, float* egrads, float* pgrads,
                       const int* inLen, const int* labLen, const Dims& d, const SparseTerms& sp,
                       const SparsePTerms& spp, hipStream_t s);
// Whether one launch covers the label axis.  A longer axis goes slice by slice, the slices adding
// up in the output array; 16-bit gradients then go through `wide` (fp32 scratch of wide_bytes,
// at least 32 frames of B * V values), a window of frames at a time, so that each value is still
// rounded once.
bool egrads_one_pass(const Dims& d);
int launch_egrads_stream(const float* E, const float* P, const float* mE, const float* mP,
                         const float* Wn, const float* deltas, float* egrads, const int* inLen,
                         const int* labLen, const Dims& d, bool accumulate,
                         const SparseTerms& sparse, hipStream_t s);
int launch_egrads_stream(const bf16_t* E, const bf16_t* P, const float* mE, const float* mP,
                         const float* Wn, const float* deltas, bf16_t* egrads, const int* inLen,
                         const int* labLen, const Dims& d, bool accumulate,
                         const SparseTerms& sparse, hipStream_t s, float* wide = nullptr,
                         size_t wide_bytes = 0);
int launch_egrads_stream(const f16_t* E, const f16_t* P, const float* mE, const float* mP,
                         const float* Wn, const float* deltas, f16_t* egrads, const int* inLen,
                         const int* labLen, const Dims& d, bool accumulate,
                         const SparseTerms& sparse, hipStream_t s, float* wide = nullptr,
                         size_t wide_bytes = 0);
int launch_pgrads_stream(const float* E, const float* P, const float* mE, const float* mP,
                         const float* Wt, const float* deltas, float* pgrads, const int* inLen,
                         const int* labLen, const Dims& d, bool accumulate,
                         const SparsePTerms& sparse, void* split_ws,
                         hipStream_t s);
int launch_pgrads_stream(const bf16_t* E, const bf16_t* P, const float* mE, const float* mP,
                         const float* Wt, const float* deltas, bf16_t* pgrads, const int* inLen,
                         const int* labLen, const Dims& d, bool accumulate,
                         const SparsePTerms& sparse, void* split_ws,
                         hipStream_t s);
int launch_pgrads_stream(const f16_t* E, const f16_t* P, const float* mE, const float* mP,
                         const float* Wt, const float* deltas, f16_t* pgrads, const int* inLen,
                         const int* labLen, const Dims& d, bool accumulate,
                         const SparsePTerms& sparse, void* split_ws,
                         hipStream_t s);

}  // namespace rnnt
