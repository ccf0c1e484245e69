// TEST INFRASTRUCTURE.  C-linkage doorway into the reference's own CPU sources, which the
// Makefile compiles from the reference tree alongside this file.  Nothing is restated here:
// every function forwards to the reference (transducer/transducer.h:3-49 with useCuda=false,
// transducer/test.h:51-113 for the two std::vector helpers).
#include <vector>

#include "test.h"
#include "transducer.h"

extern "C" {

void ref_forward(const float* E, const float* P, float* costs, float* alphas, const float* LN,
                 const int* labels, const int* inLen, const int* labLen, int B, int T, int U,
                 int V, int blank) {
  forward(E, P, costs, alphas, LN, labels, inLen, labLen, B, T, U, V, blank, false);
}

void ref_backward(const float* E, const float* P, float* eg, float* pg, float* lng,
                  const float* alphas, const float* LN, const int* labels, const int* inLen,
                  const int* labLen, int B, int T, int U, int V, int blank) {
  backward(E, P, eg, pg, lng, alphas, LN, labels, inLen, labLen, B, T, U, V, blank, false);
}

void ref_viterbi(const float* E, const float* P, const float* LN, int* labels, const int* inLen,
                 const int* labLen, int B, int T, int U, int V, int blank) {
  viterbi(E, P, LN, labels, inLen, labLen, B, T, U, V, blank, false);
}

void ref_compute_log_norms(const float* E, const float* P, float* LN, const int* inLen,
                           const int* labLen, int B, int T, int U, int V) {
  std::vector<float> e(E, E + (size_t)B * T * V), p(P, P + (size_t)B * U * V);
  std::vector<int> il(inLen, inLen + B), ll(labLen, labLen + B);
  std::vector<float> ln = computeLogNorms(e, p, il, ll, T, U, V);
  std::memcpy(LN, ln.data(), sizeof(float) * ln.size());
}

void ref_accumulate_grads(const float* E, const float* P, float* eg, float* pg,
                          const float* dalphas, const float* LN, const int* inLen,
                          const int* labLen, int B, int T, int U, int V) {
  const size_t ne = (size_t)B * T * V, np = (size_t)B * U * V, nl = (size_t)B * T * U;
  std::vector<float> e(E, E + ne), p(P, P + np), ge(eg, eg + ne), gp(pg, pg + np);
  std::vector<float> da(dalphas, dalphas + nl), ln(LN, LN + nl);
  std::vector<int> il(inLen, inLen + B), ll(labLen, labLen + B);
  accumulateGrads(e, p, ge, gp, da, ln, il, ll, T, U, V);
  std::memcpy(eg, ge.data(), sizeof(float) * ne);
  std::memcpy(pg, gp.data(), sizeof(float) * np);
}

}  // extern "C"
