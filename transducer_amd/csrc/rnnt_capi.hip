// extern "C" entry points of librnnt_hip.so (declared in include/rnnt_hip.h): argument checks,
// stream-ordered scratch, and the kernel sequences.  No torch types, no exceptions.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <atomic>
#include <mutex>

#include "../../include/rnnt_hip.h"
#include "rnnt_internal.h"

namespace rnnt {

static thread_local char g_error[512] = "";

// whether the whole-loss backward pass may form both dense gradients in one kernel
static std::atomic<int> g_fused_grads{0};

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

// Message format follows the reference's CUDA_CHECK (transducer/transducer_cuda.cu:271-278).
int check_hip(hipError_t e, const char* what, const char* file, int line) {
  if (e == hipSuccess) return kOk;
  return fail(kHipError, "[%s:%d] HIP error: %s (%s)", file, line, hipGetErrorString(e), what);
}

// ---------------------------------------------------------------- stage timing
// Optional HIP-event brackets around every kernel stage, on the stream the stage runs on.
// A single-threaded diagnostic: enable, run, read.  Off by default and free when off.
namespace prof {

enum Stage {
  kRowmax, kLse, kSkew, kGather, kAlpha, kUnskew, kWeights, kBeta, kWplanes, kEgrads, kPgrads,
  kSparse, kMaxplus, kViterbi, kClear, kYplanes, kGrads, kNumStages
};
const char* const kNames[kNumStages] = {"rowmax", "lse", "skew", "gather", "alpha", "unskew",
                                        "weights", "beta", "wplanes", "egrads", "pgrads",
                                        "sparse", "maxplus", "viterbi", "clear", "yplanes",
                                        "grads"};
constexpr int kMaxRecords = 8192;
struct Record { int stage; hipEvent_t begin, end; };

bool g_on = false;
Record g_rec[kMaxRecords];
int g_used = 0, g_created = 0;

struct Scope {
  Record* r = nullptr;
  hipStream_t s;
  Scope(int stage, hipStream_t stream) : s(stream) {
    if (!g_on || g_used == kMaxRecords) return;
    if (g_used == g_created) {
      if (hipEventCreate(&g_rec[g_created].begin) != hipSuccess) return;
      if (hipEventCreate(&g_rec[g_created].end) != hipSuccess) return;
      ++g_created;
    }
    r = &g_rec[g_used++];
    r->stage = stage;
    (void)hipEventRecord(r->begin, s);
  }
  ~Scope() {
    if (r) (void)hipEventRecord(r->end, s);
  }
};

}  // namespace prof

#define RNNT_STAGE(stage, expr)             \
  do {                                      \
    ::rnnt::prof::Scope _scope(::rnnt::prof::stage, s); \
    int _st = (expr);                       \
    if (_st != ::rnnt::kOk) return _st;     \
  } while (0)

namespace {

size_t align_up(size_t x) { return (x + 255) & ~(size_t)255; }

// The stream-ordered allocations of the entry points that take their own scratch come from a
// memory pool of the library's own, one per device, that keeps what is freed (release threshold
// at its maximum): the device's default pool hands freed memory back to the driver at the next
// synchronisation, and a caller that synchronises per call (the reference's benchmarks do) then
// pays the driver for the same blocks again on every call -- 0.1 ms of a 2.9 ms decode, 0.5 ms
// of a forward + backward through the three-call interface.  What the pool holds is the scratch
// of the largest call so far; rnnt_hip_release_scratch() returns it to the driver.
constexpr int kMaxPoolDevices = 64;
hipMemPool_t g_pool[kMaxPoolDevices];
bool g_pool_made[kMaxPoolDevices];
std::mutex g_pool_mutex;

int scratch_pool(hipMemPool_t* out) {
  int dev = 0;
  RNNT_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxPoolDevices) return fail(kInvalid, "device index %d not supported", dev);
  std::lock_guard<std::mutex> lock(g_pool_mutex);
  if (!g_pool_made[dev]) {
    hipMemPoolProps props = {};
    props.allocType = hipMemAllocationTypePinned;
    props.handleTypes = hipMemHandleTypeNone;
    props.location.type = hipMemLocationTypeDevice;
    props.location.id = dev;
    RNNT_HIP(hipMemPoolCreate(&g_pool[dev], &props));
    uint64_t keep = UINT64_MAX;
    RNNT_HIP(hipMemPoolSetAttribute(g_pool[dev], hipMemPoolAttrReleaseThreshold, &keep));
    g_pool_made[dev] = true;
  }
  *out = g_pool[dev];
  return kOk;
}

// Device scratch of one call, carved into pieces.  Either one stream-ordered allocation,
// released on the same stream when the call returns, or a fixed region that the caller of the
// constructor owns (the static array of the entry point that allocates nothing).
class Scratch {
 public:
  explicit Scratch(hipStream_t s) : stream_(s) {}
  Scratch(void* fixed, size_t capacity, const char* who)
      : stream_(nullptr), fixed_(fixed), capacity_(capacity), who_(who) {}
  ~Scratch() {
    if (base_ && !fixed_) (void)hipFreeAsync(base_, stream_);
  }
  int reserve(size_t bytes) {
    if (bytes == 0) return kOk;
    if (fixed_) {
      if (bytes > capacity_)
        return fail(kWorkspace, "%s: this problem needs %zu bytes of scratch, the built-in "
                                "array holds %zu; use the allocating entry point", who_, bytes,
                    capacity_);
      base_ = fixed_;
    } else {
      hipMemPool_t pool;
      RNNT_TRY(scratch_pool(&pool));
      RNNT_HIP(hipMallocFromPoolAsync(&base_, bytes, pool, stream_));
    }
    size_ = bytes;
    return kOk;
  }
  void* take(size_t bytes) {
    void* p = static_cast<char*>(base_) + used_;
    used_ += align_up(bytes);
    return p;
  }
  size_t used() const { return used_; }
  size_t size() const { return size_; }

 private:
  hipStream_t stream_;
  void* fixed_ = nullptr;
  size_t capacity_ = 0;
  const char* who_ = "";
  void* base_ = nullptr;
  size_t size_ = 0, used_ = 0;
};

int check_dims(int B, int T, int U, int V) {
  if (B < 0 || T < 0 || U < 0 || V < 0)
    return fail(kInvalid, "negative size (B=%d T=%d U=%d V=%d)", B, T, U, V);
  if ((long long)T * V >= (1ll << 31) || (long long)U * V >= (1ll << 31) ||
      (long long)T * U >= (1ll << 31))
    return fail(kInvalid, "one utterance's T*V, U*V or T*U exceeds 2^31 elements");
  return kOk;
}

// The reference indexes rows with `blank` unchecked (transducer/transducer_cpu.cpp:46,96); a
// value outside the vocabulary would read and write past every row, so it is refused here.
int check_blank(int V, int blank) {
  if (V > 0 && (blank < 0 || blank >= V))
    return fail(kInvalid, "blank index %d outside the vocabulary [0, %d)", blank, V);
  return kOk;
}

bool nothing_to_do(int B, int T, int U) { return B == 0 || T == 0 || U == 0; }

// Row maxima of the predictions, the Y pieces, then the streaming log-normaliser (which finds
// the emissions' per-frame reference itself); `scratch` holds lse_scratch_bytes(d).
// With `planes`, the blank / label scores the lattice recursions need are extracted on the way
// (no separate gather).
int log_norms_stages(const float* E, const float* P, float* mE, float* mP, float* LN,
                     void* scratch, const int* inLen, const int* labLen, const Dims& d,
                     hipStream_t s, const Planes* planes = nullptr, const int* labels = nullptr,
                     bool* ln_in_plane = nullptr) {
  if (ln_in_plane) *ln_in_plane = false;
  if (!scratch || !lse_stream_supported(E, d))
    return fail(kInvalid, "log-normaliser: more than 2^30 tiles of 128 frames x 128 label "
                          "positions (B=%d T=%d U=%d)", d.B, d.T, d.U);
  // one pass over E: the streaming kernel finds its own per-frame reference and leaves it in mE
  // and, with `planes`, copies the blank / label scores out of the rows as they stream by
  // (its pick list holds 1024 labels; without labels only the blank column is picked)
  if (planes && (labels == nullptr || d.U - 1 <= 1024)) {
    RNNT_STAGE(kRowmax, launch_rowmax_pick_p(P, mP, labels, labLen, *planes, d, s));
    RNNT_STAGE(kYplanes, launch_yplanes(P, mP, scratch, labLen, d, s));
    // (with the flag the caller says it only needs LN in the lattice plane)
    RNNT_STAGE(kLse, launch_lse_stream(E, mE, mP, LN, scratch, inLen, labLen, d, s, labels,
                                       planes->elS, planes->eb,
                                       ln_in_plane ? planes->lnS : nullptr));
    if (ln_in_plane) *ln_in_plane = true;
    return kOk;
  }
  RNNT_STAGE(kRowmax, launch_rowmax(P, mP, (long)d.B * d.U, d.V, d.U, labLen, 1, s));
  RNNT_STAGE(kYplanes, launch_yplanes(P, mP, scratch, labLen, d, s));
  RNNT_STAGE(kLse, launch_lse_stream(E, mE, mP, LN, scratch, inLen, labLen, d, s));
  if (planes) RNNT_STAGE(kGather, launch_gather(E, P, labels, inLen, labLen, *planes, d, s));
  return kOk;
}

struct LossWorkspace {
  Planes planes;
  float *mE, *mP, *LN, *Wn, *Wt, *bsum, *emT;
  WImages img;  // shares its memory with Wn / Wt: a backward call writes one form or the other
  void* lse_scratch;
  void* psplit;  // pgrads_split_bytes(d) bytes, or null
};

size_t loss_workspace_layout(const Dims& d, void* base, LossWorkspace* w) {
  char* c = static_cast<char*>(base);
  size_t off = 0;
  auto take = [&](size_t bytes) {
    float* p = base ? reinterpret_cast<float*>(c + off) : nullptr;
    off += align_up(bytes);
    return p;
  };
  const size_t pb = planes_bytes(d);
  void* pl = take(pb);
  if (base) carve_planes(pl, d, &w->planes);
  const size_t btu = sizeof(float) * (size_t)d.B * d.T * d.U;
  float* mE = take(sizeof(float) * (size_t)d.B * d.T);
  float* mP = take(sizeof(float) * (size_t)d.B * d.U);
  // (row-major LN: only when the log-normaliser cannot write it into the lattice plane itself,
  // i.e. with more labels than its pick list holds)
  float* LN = d.U - 1 > 1024 ? take(btu) : nullptr;
  // W for the gradient kernels: two fp32 planes, or (fused kernel) the two slab images of bf16
  // pieces, in the same memory
  const size_t wb = align_up(sizeof(float) * (size_t)d.B * wplane_tw(d.T) * wplane_up(d.U));
  const bool images = grads_fused_possible(d);
  const size_t ie = images ? align_up(WImages::e_bytes(d.B, wplane_tw(d.T))) : 0;
  const size_t ip = images ? align_up(WImages::p_bytes(d.B, wplane_tw(d.T))) : 0;
  float* Wn = take(2 * wb > ie + ip ? 2 * wb : ie + ip);
  float* Wt = Wn ? reinterpret_cast<float*>(reinterpret_cast<char*>(Wn) + wb) : nullptr;
  float* bsum = take(sizeof(float) * (size_t)d.B * d.T);
  float* emT = take(btu);  // label-move terms of egrads, [B][U][T]
  void* ys = take(lse_scratch_bytes(d));  // forward only
  void* ps = take(pgrads_split_bytes(d));  // backward only
  if (base) {
    w->mE = mE; w->mP = mP; w->LN = LN; w->Wn = Wn; w->Wt = Wt; w->bsum = bsum; w->emT = emT;
    if (images) {
      w->img.e = reinterpret_cast<unsigned*>(Wn);
      w->img.p = reinterpret_cast<unsigned*>(reinterpret_cast<char*>(Wn) + ie);
    }
    w->lse_scratch = lse_scratch_bytes(d) ? ys : nullptr;
    w->psplit = pgrads_split_bytes(d) ? ps : nullptr;
  }
  return off;
}

// cost = +inf for every utterance when the padded frame axis is empty (transducer_cpu.cpp:39-41)
__global__ void fill_kernel(float* x, float v, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) x[i] = v;
}

// Zero fill by a kernel (the whole-loss entry points enqueue kernels only, so that a caller
// may capture them into a graph; this is their degenerate T == 0 / U == 0 case).
__global__ void zero_bytes_kernel(unsigned char* x, size_t n) {
  const size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x) * 16;
  if (i + 16 <= n) {
    if ((reinterpret_cast<uintptr_t>(x) & 15) == 0) {
      *reinterpret_cast<uint4*>(x + i) = make_uint4(0, 0, 0, 0);
      return;
    }
  }
  for (size_t k = i; k < n && k < i + 16; ++k) x[k] = 0;
}

int zero_fill(void* x, size_t bytes, hipStream_t s) {
  if (x == nullptr || bytes == 0) return kOk;
  const size_t blocks = (bytes + 4095) / 4096;
  if (blocks > 0x7fffffffu) return fail(kInvalid, "array too large to clear");
  hipLaunchKernelGGL(zero_bytes_kernel, dim3((unsigned)blocks), dim3(256), 0, s,
                     static_cast<unsigned char*>(x), bytes);
  return check_hip(hipGetLastError(), "launch zero_bytes_kernel", __FILE__, __LINE__);
}

int fill(float* x, float v, int n, hipStream_t s) {
  if (n == 0) return kOk;
  hipLaunchKernelGGL(fill_kernel, dim3((n + 255) / 256), dim3(256), 0, s, x, v, n);
  return check_hip(hipGetLastError(), "launch fill_kernel", __FILE__, __LINE__);
}

// Scratch the best-path stages need (planes, the two max-plus planes, the decision table).
// `lists`: whether this call builds its table of best labels from candidate lists (asked once
// per call, so that what is reserved and what is taken agree whatever another thread sets).
size_t viterbi_scratch_bytes(const Dims& d, bool lists) {
  const size_t plane = sizeof(float) * (size_t)d.B * d.Ua * d.Dp + 64;
  return align_up(planes_bytes(d, true)) + 2 * align_up(plane) +
         align_up(viterbi_bits_bytes(d)) +
         (lists ? align_up(maxplus_lists_bytes(d)) : 0);
}

// `scratch` has viterbi_scratch_bytes(d, with_lists) left to take (one allocation per call, made by the caller
// together with whatever else it needs: the allocator calls are a visible part of a small decode).
// With `ready`, the lattice planes were carved by the caller and already hold LN and the blank
// scores (the log-normaliser left them there): no transposing copy, no gather.
template <typename TIO>
int viterbi_impl(const TIO* E, const TIO* P, const float* LN, int* labels,
                        const int* inLen, const int* labLen, const Dims& d, Scratch& scratch,
                        hipStream_t s, int plan, const Planes* ready = nullptr) {
  const bool with_lists = plan != 0;
  const size_t plane = sizeof(float) * (size_t)d.B * d.Ua * d.Dp + 64;
  Planes p;
  if (ready) p = *ready;
  else carve_planes(scratch.take(planes_bytes(d, true)), d, &p, true);
  float* bestS = static_cast<float*>(scratch.take(plane));
  float* argS = static_cast<float*>(scratch.take(plane));
  unsigned long long* bits =
      static_cast<unsigned long long*>(scratch.take(viterbi_bits_bytes(d)));
  void* lists = with_lists ? scratch.take(maxplus_lists_bytes(d)) : nullptr;
  RNNT_STAGE(kMaxplus, launch_maxplus(E, P, inLen, labLen, bestS, reinterpret_cast<int*>(argS), d,
                                      s, lists, plan == 2));
  if (!ready) {
    RNNT_STAGE(kSkew, launch_skew(LN, p.lnS, inLen, labLen, d, s));
    // blank scores only: the label planes of the gather are not needed here
    RNNT_STAGE(kGather, launch_gather(E, P, nullptr, inLen, labLen, p, d, s));
  }
  RNNT_STAGE(kViterbi, launch_viterbi(p, bestS, argS, bits, inLen, labLen, labels, d, s));
  return kOk;
}


// ---------------------------------------------------------------- 16-bit scores
int check_lowp_shape(const Dims& d, bool loss, const char* who) {
  // the blank / label terms are folded into the dense kernels' write-outs (one rounding per
  // gradient entry), which keep a list of at most 1024 labels per wavefront
  if (loss && d.U - 1 > 1024)
    return fail(kInvalid, "%s: 16-bit scores take at most 1025 label positions (U=%d)", who, d.U);
  return kOk;
}

template <typename TIO>
int lowp_loss_forward(const TIO* E, const TIO* P, const int* labels, const int* inLen,
                      const int* labLen, float* costs, void* workspace, size_t workspace_bytes,
                      int B, int T, int U, int V, int blank, rnnt_stream_t stream,
                      const char* who) {
  RNNT_TRY(check_dims(B, T, U, V));
  RNNT_TRY(check_blank(V, blank));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (B == 0) return kOk;
  if (!costs || !inLen || !labLen) return fail(kInvalid, "%s: null costs or lengths", who);
  if (nothing_to_do(B, T, U)) return fill(costs, __builtin_huge_valf(), B, s);
  if (V == 0) return fail(kInvalid, "%s: empty vocabulary", who);
  if (!E || !P || (U > 1 && !labels)) return fail(kInvalid, "%s: null array argument", who);
  if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 255))
    return fail(kInvalid, "%s: workspace must be a 256-byte aligned device pointer", who);
  if (workspace_bytes < rnnt_hip_loss_workspace_bytes(B, T, U, V))
    return fail(kWorkspace, "%s: workspace of %zu bytes, %zu needed", who, workspace_bytes,
                rnnt_hip_loss_workspace_bytes(B, T, U, V));
  const Dims d = make_dims(B, T, U, V, blank);
  RNNT_TRY(check_lowp_shape(d, true, who));
  if (!lse_stream_supported(E, d)) return fail(kInvalid, "%s: B*T*U too large", who);
  LossWorkspace w;
  loss_workspace_layout(d, workspace, &w);
  RNNT_STAGE(kRowmax, launch_rowmax_pick_p(P, w.mP, labels, labLen, w.planes, d, s));
  RNNT_STAGE(kYplanes, launch_yplanes(P, w.mP, w.lse_scratch, labLen, d, s));
  RNNT_STAGE(kLse, launch_lse_stream(E, w.mE, w.mP, w.LN, w.lse_scratch, inLen, labLen, d, s,
                                     labels, w.planes.elS, w.planes.eb, w.planes.lnS));
  RNNT_STAGE(kAlpha, launch_alpha(w.planes, inLen, labLen, costs, d, s));
  return kOk;
}

template <typename TIO>
int lowp_loss_backward(const TIO* E, const TIO* P, const int* labels, const int* inLen,
                       const int* labLen, const float* deltas, TIO* egrads, TIO* pgrads,
                       void* workspace, size_t workspace_bytes, int B, int T, int U, int V,
                       int blank, rnnt_stream_t stream, const char* who) {
  RNNT_TRY(check_dims(B, T, U, V));
  RNNT_TRY(check_blank(V, blank));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (B == 0 || V == 0) return kOk;
  if (nothing_to_do(B, T, U)) {
    RNNT_TRY(zero_fill(egrads, sizeof(TIO) * (size_t)B * T * V, s));
    RNNT_TRY(zero_fill(pgrads, sizeof(TIO) * (size_t)B * U * V, s));
    return kOk;
  }
  if (!E || !P || !egrads || !pgrads || !inLen || !labLen || (U > 1 && !labels))
    return fail(kInvalid, "%s: null array argument", who);
  if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 255))
    return fail(kInvalid, "%s: workspace must be a 256-byte aligned device pointer", who);
  if (workspace_bytes < rnnt_hip_loss_workspace_bytes(B, T, U, V))
    return fail(kWorkspace, "%s: workspace of %zu bytes, %zu needed", who, workspace_bytes,
                rnnt_hip_loss_workspace_bytes(B, T, U, V));
  const Dims d = make_dims(B, T, U, V, blank);
  RNNT_TRY(check_lowp_shape(d, true, who));
  if ((reinterpret_cast<uintptr_t>(egrads) | reinterpret_cast<uintptr_t>(pgrads)) & 1)
    return fail(kInvalid, "%s: misaligned gradient arrays", who);
  LossWorkspace w;
  loss_workspace_layout(d, workspace, &w);
  RNNT_STAGE(kWeights, launch_weights(w.planes, inLen, labLen, d, s));
  RNNT_STAGE(kBeta, launch_beta(w.planes, labels, inLen, labLen, d, s));
  // Both gradients are rounded once, from the complete fp32 value: the blank / label terms are
  // always folded into the dense kernels' write-outs here, whatever the vocabulary.  With
  // U == 1 there are no labels; the kernels then never read the list, but its pointer is what
  // switches the folding on, so any valid device pointer serves.
  const int* lab = labels ? labels : inLen;
  RNNT_STAGE(kWplanes, launch_post_beta(w.planes, w.mE, w.mP, w.Wn, w.Wt, w.bsum, w.emT, lab, inLen,
                                        labLen, d, s));
  SparseTerms sp;
  sp.emT = w.emT; sp.bsum = w.bsum; sp.labels = lab;
  SparsePTerms spp;
  spp.gB = w.planes.gB; spp.gL = w.planes.gL; spp.labels = lab;
  // a label axis of more than one slice: the slices add up in fp32, in the part of the workspace
  // that held the log-normaliser's Y pieces during the forward pass (free by now)
  RNNT_STAGE(kEgrads, launch_egrads_stream(E, P, w.mE, w.mP, w.Wn, deltas, egrads, inLen, labLen,
                                           d, false, sp, s, static_cast<float*>(w.lse_scratch),
                                           lse_scratch_bytes(d)));
  RNNT_STAGE(kPgrads, launch_pgrads_stream(E, P, w.mE, w.mP, w.Wt, deltas, pgrads, inLen, labLen,
                                           d, false, spp, w.psplit, s));
  return kOk;
}

template <typename TIO>
int lowp_viterbi_decode(const TIO* E, const TIO* P, const int* inLen, const int* labLen,
                        int* labels, int B, int T, int U, int V, int blank, rnnt_stream_t stream,
                        const char* who) {
  RNNT_TRY(check_dims(B, T, U, V));
  RNNT_TRY(check_blank(V, blank));
  if (nothing_to_do(B, T, U) || U == 1) return kOk;  // no label to emit
  if (V == 0) return fail(kInvalid, "%s: empty vocabulary", who);
  if (!E || !P || !labels || !inLen || !labLen)
    return fail(kInvalid, "%s: null array argument", who);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const Dims d = make_dims(B, T, U, V, blank);
  RNNT_TRY(check_lowp_shape(d, false, who));
  if (!lse_stream_supported(E, d)) return fail(kInvalid, "%s: B*T*U too large", who);
  Scratch scratch(s);
  const size_t yb = lse_scratch_bytes(d);
  const int plan = maxplus_plan(d);
  const bool with_lists = plan != 0;
  RNNT_TRY(scratch.reserve(align_up(sizeof(float) * (size_t)B * T) +
                           align_up(sizeof(float) * (size_t)B * U) + align_up(yb) +
                           viterbi_scratch_bytes(d, with_lists)));
  float* mE = static_cast<float*>(scratch.take(sizeof(float) * (size_t)B * T));
  float* mP = static_cast<float*>(scratch.take(sizeof(float) * (size_t)B * U));
  void* ys = scratch.take(yb);
  // LN and the blank scores go straight into the lattice planes, as in the whole-loss path
  Planes p;
  carve_planes(scratch.take(planes_bytes(d, true)), d, &p, true);
  RNNT_STAGE(kRowmax, launch_rowmax_pick_p(P, mP, nullptr, labLen, p, d, s));
  RNNT_STAGE(kYplanes, launch_yplanes(P, mP, ys, labLen, d, s));
  RNNT_STAGE(kLse, launch_lse_stream(E, mE, mP, nullptr, ys, inLen, labLen, d, s, nullptr, p.elS,
                                     p.eb, p.lnS));
  return viterbi_impl(E, P, nullptr, labels, inLen, labLen, d, scratch, s, plan, &p);
}

// The best-path decode on fp32 scores; `scratch` decides where its device scratch comes from.
int decode_fp32(const float* E, const float* P, const int* inLen, const int* labLen, int* labels,
                int B, int T, int U, int V, int blank, hipStream_t s, Scratch& scratch,
                const char* who) {
  RNNT_TRY(check_dims(B, T, U, V));
  RNNT_TRY(check_blank(V, blank));
  if (nothing_to_do(B, T, U) || U == 1) return kOk;
  if (V == 0) return fail(kInvalid, "%s: empty vocabulary", who);
  if (!E || !P || !labels || !inLen || !labLen)
    return fail(kInvalid, "%s: null array argument", who);
  const Dims d = make_dims(B, T, U, V, blank);
  if (!lse_stream_supported(E, d)) return fail(kInvalid, "%s: B*T*U too large", who);
  const size_t yb = lse_scratch_bytes(d);
  const int plan = maxplus_plan(d);
  const bool with_lists = plan != 0;
  // LN and the blank scores go straight into the lattice planes, as in the whole-loss path
  // (no row-major LN, no transposing copy, no gather)
  RNNT_TRY(scratch.reserve(align_up(sizeof(float) * (size_t)B * T) +
                           align_up(sizeof(float) * (size_t)B * U) + align_up(yb) +
                           viterbi_scratch_bytes(d, with_lists)));
  float* mE = static_cast<float*>(scratch.take(sizeof(float) * (size_t)B * T));
  float* mP = static_cast<float*>(scratch.take(sizeof(float) * (size_t)B * U));
  void* ys = scratch.take(yb);
  Planes p;
  carve_planes(scratch.take(planes_bytes(d, true)), d, &p, true);
  bool ln_in_plane = false;
  RNNT_TRY(log_norms_stages(E, P, mE, mP, nullptr, ys, inLen, labLen, d, s, &p, nullptr,
                            &ln_in_plane));
  if (!ln_in_plane) return fail(kInvalid, "%s: log-normaliser left no plane", who);
  return viterbi_impl(E, P, nullptr, labels, inLen, labLen, d, scratch, s, plan, &p);
}

// ---------------------------------------------------------------- built-in scratch
// Scratch of rnnt_hip_viterbi_decode_static: a device array that exists from the moment the
// library's code is loaded on a GPU until the process ends, so that entry point never calls an
// allocator.  `g_static_scratch` is a host-side handle, not a device address: the address is
// looked up once per device, with that device current, and only that pointer is ever used.
constexpr size_t kStaticScratchBytes = (size_t)64 << 20;
static __device__ __align__(256) unsigned char g_static_scratch[kStaticScratchBytes];
constexpr int kMaxScratchDevices = 64;
static void* g_static_scratch_ptr[kMaxScratchDevices];
static std::mutex g_static_scratch_mutex;

int static_scratch(void** out) {
  int dev = 0;
  RNNT_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxScratchDevices)
    return fail(kInvalid, "device index %d not supported", dev);
  std::lock_guard<std::mutex> lock(g_static_scratch_mutex);
  if (g_static_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    RNNT_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(g_static_scratch)));
    g_static_scratch_ptr[dev] = p;
  }
  *out = g_static_scratch_ptr[dev];
  return kOk;
}

}  // namespace
}  // namespace rnnt

using namespace rnnt;

extern "C" {

const char* rnnt_hip_last_error(void) { return g_error; }
int rnnt_hip_abi_version(void) { return 1; }

int rnnt_hip_profile_enable(int on) {
  prof::g_on = on != 0;
  if (on) prof::g_used = 0;
  return kOk;
}
int rnnt_hip_profile_stage_count(void) { return prof::kNumStages; }
const char* rnnt_hip_profile_stage_name(int i) {
  return (i >= 0 && i < prof::kNumStages) ? prof::kNames[i] : "";
}
int rnnt_hip_profile_read(double* total_ms, int* launches, int n) {
  for (int i = 0; i < n; ++i) { total_ms[i] = 0.0; launches[i] = 0; }
  for (int i = 0; i < prof::g_used; ++i) {
    prof::Record& r = prof::g_rec[i];
    RNNT_HIP(hipEventSynchronize(r.end));
    float ms = 0.0f;
    RNNT_HIP(hipEventElapsedTime(&ms, r.begin, r.end));
    if (r.stage < n) { total_ms[r.stage] += ms; launches[r.stage] += 1; }
  }
  prof::g_used = 0;
  return kOk;
}

int rnnt_hip_check_kernels(rnnt_stream_t stream) {
  hipStream_t s = static_cast<hipStream_t>(stream);
  int* flag = nullptr;
  RNNT_TRY(trouble_flag(&flag));
  RNNT_HIP(hipStreamSynchronize(s));
  int raised = 0;
  RNNT_HIP(hipMemcpy(&raised, flag, sizeof(int), hipMemcpyDeviceToHost));
  if (raised == 0) return kOk;
  raised = 0;
  RNNT_HIP(hipMemcpy(flag, &raised, sizeof(int), hipMemcpyHostToDevice));
  return fail(kHipError, "a lattice kernel gave up waiting for its neighbouring wavefront's "
                         "progress (alpha or viterbi hand-over); results of the calls since the "
                         "last check are not valid");
}

int rnnt_hip_set_spin_limit(int trips) {
  const int before = g_spin_limit;
  g_spin_limit = trips < 0 ? kDefaultSpinLimit : trips;
  return before;
}

int rnnt_hip_maxplus_table(const float* E, const float* P, const int* inLen, const int* labLen,
                           float* best, int* arg, int B, int T, int U, int V, int blank,
                           rnnt_stream_t stream) {
  RNNT_TRY(check_dims(B, T, U, V));
  RNNT_TRY(check_blank(V, blank));
  if (nothing_to_do(B, T, U)) return kOk;
  if (V == 0) return fail(kInvalid, "maxplus_table: empty vocabulary");
  if (!E || !P || !best || !arg) return fail(kInvalid, "maxplus_table: null array argument");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const Dims d = make_dims(B, T, U, V, blank);
  const size_t plane = sizeof(float) * (size_t)d.B * d.Ua * d.Dp + 64;
  const int plan = maxplus_plan(d);
  const bool with_lists = plan != 0;
  Scratch scratch(s);
  RNNT_TRY(scratch.reserve(2 * align_up(plane) +
                           (with_lists ? align_up(maxplus_lists_bytes(d)) : 0)));
  float* bestS = static_cast<float*>(scratch.take(plane));
  int* argS = static_cast<int*>(scratch.take(plane));
  void* lists = with_lists ? scratch.take(maxplus_lists_bytes(d)) : nullptr;
  RNNT_STAGE(kMaxplus, launch_maxplus(E, P, inLen, labLen, bestS, argS, d, s, lists, plan == 2));
  return launch_table_out(bestS, argS, inLen, labLen, best, arg, d, s);
}

int rnnt_hip_maxplus_tries_lists(int B, int T, int U, int V) {
  if (B <= 0 || T <= 0 || U <= 0 || V <= 0) return 0;
  return maxplus_plan(make_dims(B, T, U, V, 0)) != 0 ? 1 : 0;
}

int rnnt_hip_set_fused_grads(int mode) {
  if (mode != 0) return -1;  // switched off, see rnnt_hip_loss_backward
  return g_fused_grads.exchange(0);
}

int rnnt_hip_set_maxplus_mode(int mode) {
  if (mode < 0 || mode > 2) return fail(kInvalid, "set_maxplus_mode: mode %d (0, 1 or 2)", mode);
  set_maxplus_mode(mode);
  return kOk;
}

int rnnt_hip_libm_probe(const float* x, float* expf_out, float* log1pf_out, long n,
                        rnnt_stream_t stream) {
  if (n < 0 || (n > 0 && (!x || !expf_out || !log1pf_out)))
    return fail(kInvalid, "libm_probe: null array argument");
  return launch_libm_probe(x, expf_out, log1pf_out, n, static_cast<hipStream_t>(stream));
}

int rnnt_hip_lse_bound_check(unsigned lo_bits, unsigned hi_bits, unsigned long long* violations,
                             float* worst_ratio) {
  if (lo_bits > hi_bits || lo_bits < 0x80000000u || hi_bits > 0xff800000u || !violations ||
      !worst_ratio)
    return fail(kInvalid, "lse_bound_check: bit patterns must name floats in [-inf, -0]");
  int* words = nullptr;
  RNNT_TRY(trouble_flag(&words));
  unsigned* out = reinterpret_cast<unsigned*>(words + 32);  // two spare words of the flag array
  const unsigned zero[2] = {0u, 0u};
  RNNT_HIP(hipMemcpy(out, zero, sizeof(zero), hipMemcpyHostToDevice));
  RNNT_TRY(launch_lse_bound_check(lo_bits, hi_bits, out, nullptr));
  unsigned got[2];
  RNNT_HIP(hipMemcpy(got, out, sizeof(got), hipMemcpyDeviceToHost));
  *violations = got[0];
  float ratio;
  memcpy(&ratio, &got[1], sizeof(ratio));
  *worst_ratio = ratio;
  return kOk;
}

int rnnt_hip_chain_floor(int kind, int steps, double* ns_per_step) {
  if (kind < 0 || kind > 2 || steps < 1 || !ns_per_step)
    return fail(kInvalid, "chain_floor: kind must be 0, 1 or 2, steps positive, result non-null");
  hipEvent_t t0, t1;
  RNNT_HIP(hipEventCreate(&t0));
  RNNT_HIP(hipEventCreate(&t1));
  int st = launch_chain_floor(kind, steps, nullptr);  // warm-up (code object, clocks)
  float best = 0.0f;
  for (int rep = 0; st == kOk && rep < 5; ++rep) {
    (void)hipEventRecord(t0, nullptr);
    st = launch_chain_floor(kind, steps, nullptr);
    (void)hipEventRecord(t1, nullptr);
    if (st == kOk) st = check_hip(hipEventSynchronize(t1), "hipEventSynchronize", __FILE__, __LINE__);
    float ms = 0.0f;
    if (st == kOk) st = check_hip(hipEventElapsedTime(&ms, t0, t1), "hipEventElapsedTime", __FILE__, __LINE__);
    if (rep == 0 || ms < best) best = ms;
  }
  (void)hipEventDestroy(t0);
  (void)hipEventDestroy(t1);
  if (st != kOk) return st;
  *ns_per_step = 1.0e6 * best / steps;
  return kOk;
}

int rnnt_hip_forward(const float* E, const float* P, float* costs, float* alphas, const float* LN,
                     const int* labels, const int* inLen, const int* labLen, int B, int T, int U,
                     int V, int blank, rnnt_stream_t stream) {
  RNNT_TRY(check_dims(B, T, U, V));
  RNNT_TRY(check_blank(V, blank));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (B == 0) return kOk;
  if (!costs || !inLen || !labLen) return fail(kInvalid, "forward: null costs or lengths");
  if (nothing_to_do(B, T, U)) return fill(costs, __builtin_huge_valf(), B, s);
  if (!E || !P || !alphas || !LN || (U > 1 && !labels))
    return fail(kInvalid, "forward: null array argument");
  const Dims d = make_dims(B, T, U, V, blank);
  Scratch scratch(s);
  RNNT_TRY(scratch.reserve(planes_bytes(d)));
  Planes p;
  carve_planes(scratch.take(planes_bytes(d)), d, &p);
  RNNT_STAGE(kSkew, launch_skew(LN, p.lnS, inLen, labLen, d, s));
  RNNT_STAGE(kGather, launch_gather(E, P, labels, inLen, labLen, p, d, s));
  RNNT_STAGE(kAlpha, launch_alpha(p, inLen, labLen, costs, d, s));
  RNNT_STAGE(kUnskew, launch_unskew(p.aS, alphas, inLen, labLen, d, s));
  return kOk;
}

int rnnt_hip_backward(const float* E, const float* P, float* egrads, float* pgrads, float* lngrads,
                      const float* alphas, const float* LN, const int* labels, const int* inLen,
                      const int* labLen, int B, int T, int U, int V, int blank,
                      rnnt_stream_t stream) {
  RNNT_TRY(check_dims(B, T, U, V));
  RNNT_TRY(check_blank(V, blank));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (B == 0) return kOk;
  // transducer_cuda.cu:326-331: the library clears all three outputs itself
  {
    prof::Scope scope(prof::kClear, s);
    if (egrads && (size_t)T * V) RNNT_HIP(hipMemsetAsync(egrads, 0, sizeof(float) * (size_t)B * T * V, s));
    if (pgrads && (size_t)U * V) RNNT_HIP(hipMemsetAsync(pgrads, 0, sizeof(float) * (size_t)B * U * V, s));
    if (lngrads && (size_t)T * U) RNNT_HIP(hipMemsetAsync(lngrads, 0, sizeof(float) * (size_t)B * T * U, s));
  }
  if (nothing_to_do(B, T, U) || V == 0) return kOk;
  if (!E || !P || !egrads || !pgrads || !lngrads || !alphas || !LN || !inLen || !labLen ||
      (U > 1 && !labels))
    return fail(kInvalid, "backward: null array argument");
  const Dims d = make_dims(B, T, U, V, blank);
  Scratch scratch(s);
  const size_t bt = align_up(sizeof(float) * (size_t)B * T);
  const size_t but = align_up(sizeof(float) * (size_t)B * U * T);
  RNNT_TRY(scratch.reserve(planes_bytes(d) + bt + but));
  Planes p;
  carve_planes(scratch.take(planes_bytes(d)), d, &p);
  float* bsum = static_cast<float*>(scratch.take(bt));   // per-frame blank totals
  float* emT = static_cast<float*>(scratch.take(but));   // per-cell label-move terms
  RNNT_STAGE(kSkew, launch_skew(LN, p.lnS, inLen, labLen, d, s));
  RNNT_STAGE(kSkew, launch_skew(alphas, p.aS, inLen, labLen, d, s));
  RNNT_STAGE(kGather, launch_gather(E, P, labels, inLen, labLen, p, d, s));
  RNNT_STAGE(kWeights, launch_weights(p, inLen, labLen, d, s));
  RNNT_STAGE(kBeta, launch_beta(p, labels, inLen, labLen, d, s));
  RNNT_STAGE(kUnskew, launch_unskew(p.dS, lngrads, inLen, labLen, d, s));
  // (with U == 1 there are no labels; the kernels then never read the list)
  RNNT_STAGE(kSparse, launch_post_beta(p, nullptr, nullptr, nullptr, nullptr, bsum, emT,
                                       labels ? labels : inLen, inLen, labLen, d, s));
  RNNT_STAGE(kSparse, launch_sparse(p, bsum, emT, egrads, pgrads, labels, inLen, labLen, nullptr,
                                    false, d, s));
  return kOk;
}

int rnnt_hip_viterbi(const float* E, const float* P, const float* LN, int* labels,
                     const int* inLen, const int* labLen, int B, int T, int U, int V, int blank,
                     rnnt_stream_t stream) {
  RNNT_TRY(check_dims(B, T, U, V));
  RNNT_TRY(check_blank(V, blank));
  if (nothing_to_do(B, T, U) || U == 1) return kOk;  // no label to emit
  if (!E || !P || !LN || !labels || !inLen || !labLen)
    return fail(kInvalid, "viterbi: null array argument");
  const Dims d = make_dims(B, T, U, V, blank);
  hipStream_t s = static_cast<hipStream_t>(stream);
  Scratch scratch(s);
  const int plan = maxplus_plan(d);
  const bool with_lists = plan != 0;
  RNNT_TRY(scratch.reserve(viterbi_scratch_bytes(d, with_lists)));
  return viterbi_impl(E, P, LN, labels, inLen, labLen, d, scratch, s, plan);
}

int rnnt_hip_log_norms(const float* E, const float* P, float* LN, const int* inLen,
                       const int* labLen, int B, int T, int U, int V, rnnt_stream_t stream) {
  RNNT_TRY(check_dims(B, T, U, V));
  if (nothing_to_do(B, T, U)) return kOk;
  if (!E || !P || !LN) return fail(kInvalid, "log_norms: null array argument");
  if (V == 0) return fail(kInvalid, "log_norms: empty vocabulary");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const Dims d = make_dims(B, T, U, V, 0);
  Scratch scratch(s);
  const size_t yb = lse_stream_supported(E, d) ? lse_scratch_bytes(d) : 0;
  RNNT_TRY(scratch.reserve(align_up(sizeof(float) * (size_t)B * T) +
                           align_up(sizeof(float) * (size_t)B * U) + align_up(yb)));
  float* mE = static_cast<float*>(scratch.take(sizeof(float) * (size_t)B * T));
  float* mP = static_cast<float*>(scratch.take(sizeof(float) * (size_t)B * U));
  void* ys = yb ? scratch.take(yb) : nullptr;
  return log_norms_stages(E, P, mE, mP, LN, ys, inLen, labLen, d, s);
}

int rnnt_hip_dense_grads(const float* E, const float* P, float* egrads, float* pgrads,
                         const float* lngrads, const float* LN, const float* deltas,
                         const int* inLen, const int* labLen, int B, int T, int U, int V,
                         rnnt_stream_t stream) {
  RNNT_TRY(check_dims(B, T, U, V));
  if (nothing_to_do(B, T, U) || V == 0) return kOk;
  if (!E || !P || !egrads || !pgrads || !lngrads || !LN)
    return fail(kInvalid, "dense_grads: null array argument");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const Dims d = make_dims(B, T, U, V, 0);
  const size_t wb = sizeof(float) * (size_t)B * wplane_tw(T) * wplane_up(U);
  Scratch scratch(s);
  RNNT_TRY(scratch.reserve(align_up(sizeof(float) * (size_t)B * T) +
                           align_up(sizeof(float) * (size_t)B * U) + 2 * align_up(wb) +
                           align_up(pgrads_split_bytes(d))));
  float* mE = static_cast<float*>(scratch.take(sizeof(float) * (size_t)B * T));
  float* mP = static_cast<float*>(scratch.take(sizeof(float) * (size_t)B * U));
  float* Wn = static_cast<float*>(scratch.take(wb));
  float* Wt = static_cast<float*>(scratch.take(wb));
  void* psplit = pgrads_split_bytes(d) ? scratch.take(pgrads_split_bytes(d)) : nullptr;
  RNNT_STAGE(kRowmax, launch_rowmax(E, mE, (long)B * T, V, T, inLen, 0, s));
  RNNT_STAGE(kRowmax, launch_rowmax(P, mP, (long)B * U, V, U, labLen, 1, s));
  RNNT_STAGE(kWplanes, launch_wplanes(lngrads, LN, mE, mP, Wn, Wt, inLen, labLen, d, s));
  RNNT_STAGE(kEgrads, launch_egrads(E, P, mE, mP, Wn, deltas, egrads, inLen, labLen, d, true,
                                    SparseTerms(), s));
  RNNT_STAGE(kPgrads, launch_pgrads(E, P, mE, mP, Wt, deltas, pgrads, inLen, labLen, d, true,
                                    SparsePTerms(), psplit, s));
  return kOk;
}

size_t rnnt_hip_loss_workspace_bytes(int B, int T, int U, int V) {
  if (B <= 0 || T <= 0 || U <= 0 || V <= 0) return 256;
  const Dims d = make_dims(B, T, U, V, 0);
  return loss_workspace_layout(d, nullptr, nullptr) + 256;
}

int rnnt_hip_loss_forward(const float* E, const float* P, const int* labels, const int* inLen,
                          const int* labLen, float* costs, void* workspace, size_t workspace_bytes,
                          int B, int T, int U, int V, int blank, rnnt_stream_t stream) {
  RNNT_TRY(check_dims(B, T, U, V));
  RNNT_TRY(check_blank(V, blank));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (B == 0) return kOk;
  if (!costs || !inLen || !labLen) return fail(kInvalid, "loss_forward: null costs or lengths");
  if (nothing_to_do(B, T, U)) return fill(costs, __builtin_huge_valf(), B, s);
  if (V == 0) return fail(kInvalid, "loss_forward: empty vocabulary");
  if (!E || !P || (U > 1 && !labels)) return fail(kInvalid, "loss_forward: null array argument");
  if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 255))
    return fail(kInvalid, "loss_forward: workspace must be a 256-byte aligned device pointer");
  if (workspace_bytes < rnnt_hip_loss_workspace_bytes(B, T, U, V))
    return fail(kWorkspace, "loss_forward: workspace of %zu bytes, %zu needed", workspace_bytes,
                rnnt_hip_loss_workspace_bytes(B, T, U, V));
  const Dims d = make_dims(B, T, U, V, blank);
  LossWorkspace w;
  loss_workspace_layout(d, workspace, &w);
  bool ln_in_plane = false;
  RNNT_TRY(log_norms_stages(E, P, w.mE, w.mP, w.LN, w.lse_scratch, inLen, labLen, d, s,
                            &w.planes, labels, &ln_in_plane));
  if (!ln_in_plane) RNNT_STAGE(kSkew, launch_skew(w.LN, w.planes.lnS, inLen, labLen, d, s));
  RNNT_STAGE(kAlpha, launch_alpha(w.planes, inLen, labLen, costs, d, s));
  return kOk;
}

int rnnt_hip_loss_backward(const float* E, const float* P, const int* labels, const int* inLen,
                           const int* labLen, const float* deltas, float* egrads, float* pgrads,
                           void* workspace, size_t workspace_bytes, int B, int T, int U, int V,
                           int blank, rnnt_stream_t stream) {
  RNNT_TRY(check_dims(B, T, U, V));
  RNNT_TRY(check_blank(V, blank));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (B == 0 || V == 0) return kOk;
  if (nothing_to_do(B, T, U)) {
    RNNT_TRY(zero_fill(egrads, sizeof(float) * (size_t)B * T * V, s));
    RNNT_TRY(zero_fill(pgrads, sizeof(float) * (size_t)B * U * V, s));
    return kOk;
  }
  if (!E || !P || !egrads || !pgrads || !inLen || !labLen || (U > 1 && !labels))
    return fail(kInvalid, "loss_backward: null array argument");
  if (!workspace || (reinterpret_cast<uintptr_t>(workspace) & 255))
    return fail(kInvalid, "loss_backward: workspace must be a 256-byte aligned device pointer");
  if (workspace_bytes < rnnt_hip_loss_workspace_bytes(B, T, U, V))
    return fail(kWorkspace, "loss_backward: workspace of %zu bytes, %zu needed", workspace_bytes,
                rnnt_hip_loss_workspace_bytes(B, T, U, V));
  const Dims d = make_dims(B, T, U, V, blank);
  LossWorkspace w;
  loss_workspace_layout(d, workspace, &w);
  RNNT_STAGE(kWeights, launch_weights(w.planes, inLen, labLen, d, s));
  RNNT_STAGE(kBeta, launch_beta(w.planes, labels, inLen, labLen, d, s));

  // The blank/label terms of egrads are folded into the dense kernel's write-out (a scatter
  // afterwards would touch one cache line of the 2.5 GB array per lattice cell).
  // (not with a small vocabulary: many labels then fall into one wavefront's 32 columns and
  // their terms queue up in the dense kernel -- B=8 V=100: 0.17 ms folded, 0.03 + 0.04 ms
  // scattered; from V=1000 on folding is level or ahead)
  // (and not with more than 1024 labels: the dense kernel's per-wavefront match list holds
  // that many)
  // The one-kernel form of the two gradients (rnnt_fused.hip) is switched off: at the headline
  // shape it left NaN entries in pgrads on one input and made an illegal memory access on
  // another, and the cause has not been found.  rnnt_hip_set_fused_grads refuses to switch it
  // on, so use_fused is always false here.
  const int fused_mode = g_fused_grads.load();
  const bool use_fused = labels != nullptr && grads_fused_possible(d) &&
                         (fused_mode == 2 || (fused_mode == 1 && grads_fused_pays(d)));
  const bool fold = labels != nullptr && (d.V >= 512 || use_fused) && d.U - 1 <= 1024;
  RNNT_STAGE(kWplanes, launch_post_beta(w.planes, w.mE, w.mP, w.Wn, w.Wt,
                                        w.bsum, w.emT, labels ? labels : inLen, inLen, labLen, d, s,
                                        use_fused ? w.img : WImages()));
  SparseTerms sp;
  if (fold) { sp.emT = w.emT; sp.bsum = w.bsum; sp.labels = labels; }
  // pgrads always takes its blank / label totals in its write-out (the same two fp32 operations
  // the scatter kernel would do afterwards, so the same bits, and no extra launch)
  SparsePTerms spp;
  spp.gB = w.planes.gB; spp.gL = w.planes.gL; spp.labels = labels;
  if (use_fused) {
    // one walk over the frames for both gradients: each row of E is read once
    RNNT_STAGE(kGrads, launch_grads_fused(E, P, w.mE, w.mP, w.img, deltas, egrads, pgrads,
                                          inLen, labLen, d, sp, spp, s));
    return kOk;
  }
  RNNT_STAGE(kEgrads, launch_egrads(E, P, w.mE, w.mP, w.Wn, deltas, egrads, inLen, labLen, d, false,
                                    sp, s));
  RNNT_STAGE(kPgrads, launch_pgrads(E, P, w.mE, w.mP, w.Wt, deltas, pgrads, inLen, labLen, d, false,
                                    spp, w.psplit, s));
  if (!fold)
    RNNT_STAGE(kSparse, launch_sparse(w.planes, w.bsum, w.emT, egrads, nullptr, labels, inLen,
                                      labLen, deltas, true, d, s));
  return kOk;
}

// 16-bit scores (bf16, fp16): every launcher below exists for all three element types.  The three entry
// points per type are thin wrappers around the templates above.
#define RNNT_LOWP_ENTRY_POINTS(SUFFIX, TIO)                                                       \
  int rnnt_hip_loss_forward_##SUFFIX(const uint16_t* E, const uint16_t* P, const int* labels,     \
                                     const int* inLen, const int* labLen, float* costs,           \
                                     void* workspace, size_t workspace_bytes, int B, int T,       \
                                     int U, int V, int blank, rnnt_stream_t stream) {             \
    return lowp_loss_forward(reinterpret_cast<const TIO*>(E), reinterpret_cast<const TIO*>(P),    \
                             labels, inLen, labLen, costs, workspace, workspace_bytes, B, T, U,   \
                             V, blank, stream, "loss_forward_" #SUFFIX);                          \
  }                                                                                               \
  int rnnt_hip_loss_backward_##SUFFIX(const uint16_t* E, const uint16_t* P, const int* labels,    \
                                      const int* inLen, const int* labLen, const float* deltas,   \
                                      uint16_t* egrads, uint16_t* pgrads, void* workspace,        \
                                      size_t workspace_bytes, int B, int T, int U, int V,         \
                                      int blank, rnnt_stream_t stream) {                          \
    return lowp_loss_backward(reinterpret_cast<const TIO*>(E), reinterpret_cast<const TIO*>(P),   \
                              labels, inLen, labLen, deltas, reinterpret_cast<TIO*>(egrads),      \
                              reinterpret_cast<TIO*>(pgrads), workspace, workspace_bytes, B, T,   \
                              U, V, blank, stream, "loss_backward_" #SUFFIX);                     \
  }                                                                                               \
  int rnnt_hip_viterbi_decode_##SUFFIX(const uint16_t* E, const uint16_t* P, const int* inLen,    \
                                       const int* labLen, int* labels, int B, int T, int U,       \
                                       int V, int blank, rnnt_stream_t stream) {                  \
    return lowp_viterbi_decode(reinterpret_cast<const TIO*>(E), reinterpret_cast<const TIO*>(P),  \
                               inLen, labLen, labels, B, T, U, V, blank, stream,                  \
                               "viterbi_decode_" #SUFFIX);                                        \
  }
RNNT_LOWP_ENTRY_POINTS(bf16, bf16_t)
RNNT_LOWP_ENTRY_POINTS(f16, f16_t)
#undef RNNT_LOWP_ENTRY_POINTS

int rnnt_hip_viterbi_decode(const float* E, const float* P, const int* inLen, const int* labLen,
                            int* labels, int B, int T, int U, int V, int blank,
                            rnnt_stream_t stream) {
  hipStream_t s = static_cast<hipStream_t>(stream);
  Scratch scratch(s);
  return decode_fp32(E, P, inLen, labLen, labels, B, T, U, V, blank, s, scratch, "viterbi_decode");
}

int rnnt_hip_viterbi_decode_static(const float* E, const float* P, const int* inLen,
                                   const int* labLen, int* labels, int B, int T, int U, int V,
                                   int blank, rnnt_stream_t stream) {
  hipStream_t s = static_cast<hipStream_t>(stream);
  void* base = nullptr;
  RNNT_TRY(static_scratch(&base));
  Scratch scratch(base, kStaticScratchBytes, "viterbi_decode_static");
  return decode_fp32(E, P, inLen, labLen, labels, B, T, U, V, blank, s, scratch,
                     "viterbi_decode_static");
}

size_t rnnt_hip_static_scratch_bytes(void) { return kStaticScratchBytes; }

int rnnt_hip_release_scratch(void) {
  int dev = 0;
  RNNT_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxPoolDevices) return fail(kInvalid, "device index %d not supported", dev);
  std::lock_guard<std::mutex> lock(g_pool_mutex);
  if (g_pool_made[dev]) RNNT_HIP(hipMemPoolTrimTo(g_pool[dev], 0));
  return kOk;
}

}  // extern "C"
