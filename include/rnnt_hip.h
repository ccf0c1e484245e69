/*
 * C interface of librnnt_hip.so: the RNN-T loss hot path on one MI355X (gfx950).
 *
 * Every pointer is a DEVICE pointer on the current HIP device unless stated otherwise; the
 * caller owns all inputs and outputs.  Arrays are contiguous row-major with the reference's
 * shapes (transducer/transducer.h:3-49):
 *     emissions   float [B, T, V]          predictions float [B, U, V]   (U = longest label + 1)
 *     labels      int   [B, U-1]           input_lengths, label_lengths  int [B]
 *     log_norms, alphas, lngrads  float [B, T, U]     costs float [B]
 * `stream` is a hipStream_t (NULL = the null stream, which is what the reference uses,
 * transducer/transducer_cuda.cu:294-387).  Calls enqueue work and return without waiting.
 *
 * Return value: 0 on success, otherwise one of the RNNT_* codes below with a message available
 * from rnnt_hip_last_error() on the calling thread.
 */
#ifndef RNNT_HIP_H_
#define RNNT_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* rnnt_stream_t;

enum {
  RNNT_OK = 0,
  RNNT_INVALID_ARGUMENT = 1, /* bad sizes or a missing pointer */
  RNNT_HIP_FAILURE = 2,      /* a HIP runtime call failed; message holds "[file:line] HIP error: ..." */
  RNNT_WORKSPACE_TOO_SMALL = 3
};

const char* rnnt_hip_last_error(void);
int rnnt_hip_abi_version(void);

/* ---- the three entry points of the reference, device side ------------------------------- */

/* Replaces cuda::forward (transducer/transducer_cuda.h:14-27, transducer_cuda.cu:280-307):
 * alpha recursion with caller-supplied log_norms.  Writes costs[B] and the alphas of the cells
 * inside each utterance's (input_length, label_length+1) extent; other cells are untouched.
 * An utterance with input_length 0 gets cost +inf. */
int rnnt_hip_forward(const float* emissions, const float* predictions, float* costs,
                     float* alphas, const float* log_norms, const int* labels,
                     const int* input_lengths, const int* label_lengths, int B, int T, int U,
                     int V, int blank, rnnt_stream_t stream);

/* Replaces cuda::backward (transducer/transducer_cuda.h:29-44, transducer_cuda.cu:309-347):
 * zero-fills egrads, pgrads and lngrads, then writes lngrads = d cost / d log_norms and the
 * sparse blank/label terms of egrads and pgrads.
 * Like the reference it clears its outputs with memset operations (hipMemsetAsync) and, like
 * rnnt_hip_forward, rnnt_hip_viterbi, rnnt_hip_log_norms, rnnt_hip_dense_grads and
 * rnnt_hip_viterbi_decode*, takes its scratch from the stream-ordered allocator
 * (hipMallocAsync / hipFreeAsync on `stream`): none of these calls can be captured into a HIP
 * graph.  The capturable entry points are rnnt_hip_loss_forward / rnnt_hip_loss_backward and
 * their _bf16 / _f16 forms (kernels only, all memory in the caller's workspace), and
 * rnnt_hip_viterbi_decode_static (kernels only, built-in scratch). */
int rnnt_hip_backward(const float* emissions, const float* predictions, float* egrads,
                      float* pgrads, float* lngrads, const float* alphas, const float* log_norms,
                      const int* labels, const int* input_lengths, const int* label_lengths,
                      int B, int T, int U, int V, int blank, rnnt_stream_t stream);

/* Replaces cuda::viterbi (transducer/transducer_cuda.h:46-57, transducer_cuda.cu:349-388):
 * best label sequence of the given lengths with caller-supplied log_norms.  Writes the first
 * label_lengths[b] entries of labels[b]; the rest are untouched.  Pointers may be NULL when
 * T == 0, labels may be NULL when U == 1 (transducer/test.cpp:229-257). */
int rnnt_hip_viterbi(const float* emissions, const float* predictions, const float* log_norms,
                     int* labels, const int* input_lengths, const int* label_lengths, int B,
                     int T, int U, int V, int blank, rnnt_stream_t stream);

/* ---- the parts the reference computes with torch ops ------------------------------------ */

/* Replaces transducer/torch_binding.py:35-40 (and :162-167):
 * log_norms[b,t,u] = log sum_v exp(emissions[b,t,v] + predictions[b,u,v]).
 * input_lengths / label_lengths may be NULL (every cell is computed, as torch does); when given,
 * cells outside an utterance's extent are written as 0 (transducer/test.h:51-80). */
int rnnt_hip_log_norms(const float* emissions, const float* predictions, float* log_norms,
                       const int* input_lengths, const int* label_lengths, int B, int T, int U,
                       int V, rnnt_stream_t stream);

/* Replaces transducer/torch_binding.py:85-89: adds the dense softmax part
 * sum_u lngrads[b,t,u]*softmax(b,t,u)[v] (resp. sum_t) to what egrads / pgrads hold (the sparse
 * terms rnnt_hip_backward left there) and multiplies the result by deltas[b].
 * deltas may be NULL (= 1).  Frames and label positions outside an utterance stay exactly 0. */
int rnnt_hip_dense_grads(const float* emissions, const float* predictions, float* egrads,
                         float* pgrads, const float* lngrads, const float* log_norms,
                         const float* deltas, const int* input_lengths, const int* label_lengths,
                         int B, int T, int U, int V, rnnt_stream_t stream);

/* ---- whole loss, as TransducerLoss uses it ---------------------------------------------- */

/* Device bytes rnnt_hip_loss_forward/backward need between them: O(B*T*U) lattice planes,
 * O(B*(T+U)) vectors, and one O(B*U*V) entry -- the bf16 pieces of exp(predictions - row
 * maximum), 1.5 times the bytes of `predictions` with U rounded up to 32 (245 MB of the 575 MB
 * at B=32, T=2000, U=101, V=10000).  No entry of the size of `emissions`. */
size_t rnnt_hip_loss_workspace_bytes(int B, int T, int U, int V);

/* Replaces Transducer.forward (transducer/torch_binding.py:25-58): log-normaliser + alpha.
 * `workspace` (>= rnnt_hip_loss_workspace_bytes, 256-byte aligned) must stay untouched until
 * the matching rnnt_hip_loss_backward has run; it plays the role of the tensors the reference
 * saves for backward, without any [B,T,V]-sized entry. */
int rnnt_hip_loss_forward(const float* emissions, const float* predictions, const int* labels,
                          const int* input_lengths, const int* label_lengths, float* costs,
                          void* workspace, size_t workspace_bytes, int B, int T, int U, int V,
                          int blank, rnnt_stream_t stream);

/* Replaces Transducer.backward (transducer/torch_binding.py:60-90): full egrads[B,T,V] and
 * pgrads[B,U,V] (sparse + dense parts, times deltas[b]); every element is written. */
int rnnt_hip_loss_backward(const float* emissions, const float* predictions, const int* labels,
                           const int* input_lengths, const int* label_lengths,
                           const float* deltas, float* egrads, float* pgrads, void* workspace,
                           size_t workspace_bytes, int B, int T, int U, int V, int blank,
                           rnnt_stream_t stream);

/* The same calls for 16-bit scores and gradients: bf16 (the 16 high bits of an fp32, as
 * torch.bfloat16 stores them) and fp16 (IEEE binary16, torch.float16).  No counterpart in the
 * reference, which refuses anything but float32 (transducer/torch_binding.py:195-201): these are
 * for a caller whose projection layers emit 16-bit logits, and they halve the traffic of the two
 * [B,T,V] arrays.  A score converts to fp32 exactly and all arithmetic is the fp32 path's; each
 * gradient element is the fp32 result (dense + blank/label terms, times deltas[b]) rounded once
 * to nearest-even (an fp16 gradient past 65504 becomes infinity).  A label axis of more than
 * 112 positions is contracted in slices that add up in fp32 (in the workspace, a window of frames
 * at a time) before the one rounding; the loss takes at most 1025 label positions (U <= 1025) in
 * these types and refuses more with an error.  Any V; 16-byte loads are
 * used when V is a multiple of 8 and the arrays are 16-byte aligned.  Workspace as for the fp32
 * calls.  The best path of
 * rnnt_hip_viterbi_decode_* is the one rnnt_hip_viterbi_decode finds on the same values. */
int rnnt_hip_loss_forward_bf16(const uint16_t* emissions, const uint16_t* predictions,
                               const int* labels, const int* input_lengths,
                               const int* label_lengths, float* costs, void* workspace,
                               size_t workspace_bytes, int B, int T, int U, int V, int blank,
                               rnnt_stream_t stream);
int rnnt_hip_loss_backward_bf16(const uint16_t* emissions, const uint16_t* predictions,
                                const int* labels, const int* input_lengths,
                                const int* label_lengths, const float* deltas, uint16_t* egrads,
                                uint16_t* pgrads, void* workspace, size_t workspace_bytes, int B,
                                int T, int U, int V, int blank, rnnt_stream_t stream);
int rnnt_hip_viterbi_decode_bf16(const uint16_t* emissions, const uint16_t* predictions,
                                 const int* input_lengths, const int* label_lengths, int* labels,
                                 int B, int T, int U, int V, int blank, rnnt_stream_t stream);
int rnnt_hip_loss_forward_f16(const uint16_t* emissions, const uint16_t* predictions,
                              const int* labels, const int* input_lengths,
                              const int* label_lengths, float* costs, void* workspace,
                              size_t workspace_bytes, int B, int T, int U, int V, int blank,
                              rnnt_stream_t stream);
int rnnt_hip_loss_backward_f16(const uint16_t* emissions, const uint16_t* predictions,
                               const int* labels, const int* input_lengths,
                               const int* label_lengths, const float* deltas, uint16_t* egrads,
                               uint16_t* pgrads, void* workspace, size_t workspace_bytes, int B,
                               int T, int U, int V, int blank, rnnt_stream_t stream);
int rnnt_hip_viterbi_decode_f16(const uint16_t* emissions, const uint16_t* predictions,
                                const int* input_lengths, const int* label_lengths, int* labels,
                                int B, int T, int U, int V, int blank, rnnt_stream_t stream);

/* Replaces TransducerLoss.viterbi (transducer/torch_binding.py:130-177): log-normaliser +
 * best path.  labels is int [B, U-1]. */
int rnnt_hip_viterbi_decode(const float* emissions, const float* predictions,
                            const int* input_lengths, const int* label_lengths, int* labels,
                            int B, int T, int U, int V, int blank, rnnt_stream_t stream);

/* rnnt_hip_viterbi_decode for callers that cannot allocate (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference, whose
 * viterbi allocates and frees its scratch on every call (transducer/transducer_cuda.cu:364-369,
 * 386-387).  Same arguments, same result; all scratch lives in an array built into the library
 * (rnnt_hip_static_scratch_bytes() bytes, held on every GPU the library runs on until the
 * process ends), and the call makes no hipMalloc / hipFree / hipMemset of any kind.  A problem
 * whose scratch does not fit is refused with RNNT_WORKSPACE_TOO_SMALL (one utterance of the
 * headline shape, T=2000 U=101 V=10000, needs 16 MB of the 64).  Every call on a GPU uses that
 * GPU's one array: calls that overlap on one GPU (two streams, two threads) race; calls queued
 * on one stream do not.  The array's address is looked up on the first call on each device, so
 * make that first call outside any graph capture. */
int rnnt_hip_viterbi_decode_static(const float* emissions, const float* predictions,
                                   const int* input_lengths, const int* label_lengths,
                                   int* labels, int B, int T, int U, int V, int blank,
                                   rnnt_stream_t stream);
size_t rnnt_hip_static_scratch_bytes(void);

/* The entry points that take their own scratch (rnnt_hip_forward, _backward, _viterbi,
 * _log_norms, _dense_grads, _viterbi_decode*, _maxplus_table) allocate it stream-ordered, as the
 * reference's viterbi does (transducer/transducer_cuda.cu:364-369, 386-387), from a memory pool of
 * the library's own that keeps freed blocks for the next call: the scratch of the largest call so
 * far stays reserved on the device.  This hands it back to the driver (current device; call it
 * when no such call is in flight).  No counterpart in the reference. */
int rnnt_hip_release_scratch(void);

/* ---- stage timing (diagnostic; no counterpart in the reference, whose only instrumentation
 * is wall-clock loops in transducer/benchmark.cpp:21-34) ---------------------------------- */

/* When enabled, every kernel stage of the calls above is bracketed with HIP events on the
 * stream it runs on.  Not thread-safe; meant for one benchmarking thread. */
int rnnt_hip_profile_enable(int on);
int rnnt_hip_profile_stage_count(void);
const char* rnnt_hip_profile_stage_name(int stage);
/* Waits for the recorded events, writes per-stage total milliseconds and launch counts into
 * the first n entries of the two HOST arrays, and clears the record. */
int rnnt_hip_profile_read(double* total_ms, int* launches, int n);

/* ---- diagnostics of the lattice walks (no counterpart in the reference) ------------------ */

/* The lattice walks deal a long label axis to several wavefronts of a workgroup (from 257
 * label positions in a small batch the alpha and dalpha walks also to several workgroups); each
 * waits, with a trip bound, for what its neighbour hands over.  Should the bound ever run out
 * the kernel still finishes, with invalid results, and raises a flag on its device.  This call waits for `stream`, reads the current device's flag and clears it:
 * RNNT_OK if no kernel gave up since the last check, else RNNT_HIP_FAILURE with a message.
 * (The reference's kernels synchronise with __syncthreads and cannot hang this way,
 * transducer/transducer_cuda.cu:65-90.) */
int rnnt_hip_check_kernels(rnnt_stream_t stream);
/* Sets the trip bound (negative: back to the default) and returns the previous one.  For
 * tests of the give-up path: with 0 the upper wavefront gives up at its first unmet wait. */
int rnnt_hip_set_spin_limit(int trips);

/* How the best-path calls find best[t,u] = max over v != blank of E[t,v] + P[u,v] and its
 * lowest index (transducer/transducer_cpu.cpp:158-171; the reference's device kernel scans every
 * column per cell, transducer/transducer_cuda.cu:178-207).
 *   0 (default): over every column, except for vocabularies of 3000 to about 17400 entries with
 *      U x V of 250000 or more (say 33 label positions at 10000 entries, 101 at 3000): there
 *      each frame and each label position first gets a short list of its largest scores,
 *      a cell is settled from the two lists where a bound proves that no other column can win,
 *      and the remaining cells are evaluated over every column; the call looks at a sample of
 *      the cells first, takes lists half as long again if too many of them fail the bound
 *      (scores with a hard upper edge, such as uniform ones, do), and goes back to every column
 *      if too many fail with those as well;
 *   1: over every column always;
 *   2: lists for every vocabulary of up to 17408 entries, without the sample (for tests).
 * The labels returned are the same in every mode; the setting is process-wide.  No counterpart
 * in the reference. */
int rnnt_hip_set_maxplus_mode(int mode);
/* rnnt_hip_loss_backward forms the two dense gradients with two kernels, each of which reads
 * the emissions.  A one-kernel form that reads them once (both gradients from one walk over
 * the frames, transducer_amd/csrc/rnnt_fused.hip) exists for 2 to 112 label positions but is
 * SWITCHED OFF: it measured level with the two kernels and then faulted at the headline shape
 * for a reason not yet found.  mode 0 (the two kernels) returns the previous setting, 0; any
 * other mode is refused with -1 and changes nothing.  No counterpart in the reference (which
 * leaves both products to torch.bmm, transducer/torch_binding.py:85-89). */
int rnnt_hip_set_fused_grads(int mode);
/* 1 if a best-path call of this shape starts on the list path under the current mode (it may
 * still turn back after looking at a sample of the cells), else 0. */
int rnnt_hip_maxplus_tries_lists(int B, int T, int U, int V);
/* The table itself, for tests of the two ways of building it: best[b][t][u] and arg[b][t][u]
 * ([B][T][U]; -inf and -1 outside an utterance's T_b x U_b cells).  fp32 scores; scratch from
 * the stream-ordered allocator. */
int rnnt_hip_maxplus_table(const float* emissions, const float* predictions,
                           const int* input_lengths, const int* label_lengths, float* best,
                           int* arg, int B, int T, int U, int V, int blank, rnnt_stream_t stream);

/* The lattice kernels' expf and log1pf, which restate the C library's (glibc 2.35, the one the
 * reference's std::exp / std::log1p resolve to, transducer/transducer_cpu.cpp:16-24,124-135) so
 * that alphas and transition weights carry the reference's bits: expf_out[i] = expf(x[i]),
 * log1pf_out[i] = log1pf(x[i]) for n device floats (log1pf for x >= 0 only).  For tests that
 * hold them to the host's library. */
int rnnt_hip_libm_probe(const float* x, float* expf_out, float* log1pf_out, long n,
                        rnnt_stream_t stream);

/* The alpha walk forms log(exp(a) + exp(b)) on the hardware exp/log units and keeps that
 * sum only where it can show that the library's sum rounds to the same float (otherwise the
 * lane takes the library's algorithm).  The proof rests on a bound of the fast value's distance
 * from log1pf(expf(d)), d = -|a - b|.  This call checks that bound for EVERY float d whose bit
 * pattern lies in [lo_bits, hi_bits] (0x80000000 = -0 ... 0xff800000 = -inf; the whole range
 * takes a fraction of a second) on the current device, synchronously: *violations = patterns
 * where the bound fails (must be 0), *worst_ratio = largest distance / bound seen. */
int rnnt_hip_lse_bound_check(unsigned lo_bits, unsigned hi_bits, unsigned long long* violations,
                             float* worst_ratio);

/* Latency floor of one step of a lattice walk: runs `steps` steps of the bare dependent chain
 * of one cell (kind 0: alpha -- hand-over, checked fast log-sum-exp with no lane falling back,
 * the three additions of a move; kind 1: dalpha -- hand-over, two multiplies, an add; kind 2:
 * kind 0 with every lane on the library's expf/log1pf) on a single wavefront with every operand in
 * registers, times it with HIP events on the null stream (best of five) and writes nanoseconds
 * per step to the HOST double.  The measured walks are reported against this floor
 * (transducer/transducer_cuda.cu:65-90,141-175 are the loops it bounds). */
int rnnt_hip_chain_floor(int kind, int steps, double* ns_per_step);

#ifdef __cplusplus
}
#endif

#endif /* RNNT_HIP_H_ */
