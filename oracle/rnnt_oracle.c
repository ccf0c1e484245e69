/*
 * TEST INFRASTRUCTURE -- not part of the product library.
 *
 * CPU oracle for the RNN-T loss hot path (log-normaliser, alpha recursion, dalpha recursion
 * with the sparse blank/label gradient terms, dense gradient accumulation, viterbi best path).
 * It restates the algorithm of awni/transducer's CPU backend and test helpers
 * (transducer/transducer_cpu.cpp, transducer/test.h:51-113, transducer/torch_binding.py:35-40,
 * 85-89); the body lives in rnnt_oracle_impl.inc and is instantiated for float and double.
 *
 * Exported names: orc_<function>_f32 / orc_<function>_f64.  All arrays are contiguous
 * row-major: E[B,maxT,V], P[B,maxU,V], labels[B,maxU-1], LN/alphas/lngrads[B,maxT,maxU].
 * maxU is the prediction length, i.e. longest label + 1.
 *
 * Build with -ffp-contract=off so that a*b+c is never fused: the fp32 instance must round
 * exactly like the reference compiled the same way.
 *
 * How each function is pinned (none is "parity unpinned"):
 *   orc_forward/backward/viterbi_f32 and orc_log_norms_naive/accumulate_grads_f32 are compared
 *   bit for bit with the reference's own sources compiled into oracle/_ref (where that build
 *   exists) on the reference's golden vectors, a seeded ragged grid, and config-1 inputs; and
 *   in every environment against the golden literals of transducer/test.cpp:92-226,259-308,
 *   the closed form of tinyTest, brute-force path enumeration, and finite differences.
 *   orc_log_norms_sep / orc_dense_grads_sep are compared with the naive forms (same
 *   mathematics, different summation) and with the fp64 instance.
 */
#include <math.h>
#include <stdlib.h>
#include <string.h>

#define CAT2(a, b) a##b
#define CAT(a, b) CAT2(a, b)

#define REAL float
#define FN(name) CAT(name, _f32)
#define REXP expf
#define RLOG logf
#define RLOG1P log1pf
#define RABS fabsf
#include "rnnt_oracle_impl.inc"
#undef REAL
#undef FN
#undef REXP
#undef RLOG
#undef RLOG1P
#undef RABS

#define REAL double
#define FN(name) CAT(name, _f64)
#define REXP exp
#define RLOG log
#define RLOG1P log1p
#define RABS fabs
#include "rnnt_oracle_impl.inc"
#undef REAL
#undef FN
#undef REXP
#undef RLOG
#undef RLOG1P
#undef RABS

/* fp64 log-sum-exp of fp32 inputs: the "truth" the device log-normaliser is gated against.
 * Joint max, compensated by nothing -- plain fp64 is ~9 digits beyond fp32 here.
 * valid cells only when lengths are given (NULL = every cell). */
void orc_log_norms_truth(const float* E, const float* P, double* LN, const int* inLen,
                         const int* labLen, int B, int maxT, int maxU, int V) {
  memset(LN, 0, sizeof(double) * (size_t)B * maxT * maxU);
#pragma omp parallel for
  for (int b = 0; b < B; ++b) {
    const int T = inLen ? inLen[b] : maxT, U = labLen ? labLen[b] + 1 : maxU;
    for (int t = 0; t < T; ++t)
      for (int u = 0; u < U; ++u) {
        const float* e = E + ((size_t)b * maxT + t) * V;
        const float* p = P + ((size_t)b * maxU + u) * V;
        double top = -INFINITY;
        for (int v = 0; v < V; ++v) { const double s = (double)e[v] + (double)p[v]; top = top > s ? top : s; }
        double acc = 0;
        for (int v = 0; v < V; ++v) acc += exp(((double)e[v] + (double)p[v]) - top);
        LN[((size_t)b * maxT + t) * maxU + u] = log(acc) + top;
      }
  }
}

/* max-plus table used by the viterbi tests: best[b,t,u], arg[b,t,u] over v != blank of
 * E[t,v]+P[u,v] in fp32, lowest index on ties (transducer/transducer_cpu.cpp:158-171). */
void orc_best_labels_f32_table(const float* E, const float* P, float* best, int* arg,
                               const int* inLen, const int* labLen, int B, int maxT, int maxU,
                               int V, int blank) {
#pragma omp parallel for
  for (int b = 0; b < B; ++b) {
    const int T = inLen ? inLen[b] : maxT, U = labLen ? labLen[b] + 1 : maxU;
    for (int t = 0; t < T; ++t)
      for (int u = 0; u < U; ++u) {
        const size_t c = ((size_t)b * maxT + t) * maxU + u;
        best[c] = best_label_f32(E + ((size_t)b * maxT + t) * V, P + ((size_t)b * maxU + u) * V,
                                 V, blank, &arg[c]);
      }
  }
}

/* The C library's expf / log1pf elementwise: what the reference's std::exp / std::log1p resolve
 * to on floats (transducer/transducer_cpu.cpp:16-24).  The device's restatements of the two are
 * held to these bit for bit. */
void orc_libm_expf(const float* x, float* y, long n) {
#pragma omp parallel for
  for (long i = 0; i < n; ++i) y[i] = expf(x[i]);
}
void orc_libm_log1pf(const float* x, float* y, long n) {
#pragma omp parallel for
  for (long i = 0; i < n; ++i) y[i] = log1pf(x[i]);
}
