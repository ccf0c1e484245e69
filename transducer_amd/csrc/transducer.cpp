// The reference's C++ interface (include/transducer.h) over the C interface of librnnt_hip.so:
// status codes become the exception types the reference throws (transducer/transducer.cpp:41,
// transducer/transducer_cuda.cu:271-278).
#include "transducer.h"

#include <stdexcept>
#include <string>

#include "rnnt_hip.h"

namespace {

void require_device(bool useCuda) {
  if (!useCuda) throw std::invalid_argument("Transducer not built with the CPU backend.");
}

void raise_on(int status) {
  if (status == RNNT_OK) return;
  const std::string msg = rnnt_hip_last_error();
  if (status == RNNT_HIP_FAILURE) throw std::runtime_error(msg);
  throw std::invalid_argument(msg);
}

}  // namespace

void forward(const float* emissions, const float* predictions, float* costs, float* alphas,
             const float* logNorms, const int* labels, const int* inputLengths,
             const int* labelLengths, int batchSize, int maxInputLength, int maxLabelLength,
             int alphabetSize, int blank, bool useCuda) {
  require_device(useCuda);
  raise_on(rnnt_hip_forward(emissions, predictions, costs, alphas, logNorms, labels, inputLengths,
                            labelLengths, batchSize, maxInputLength, maxLabelLength, alphabetSize,
                            blank, nullptr));
}

void backward(const float* emissions, const float* predictions, float* egrads, float* pgrads,
              float* lngrads, const float* alphas, const float* logNorms, const int* labels,
              const int* inputLengths, const int* labelLengths, int batchSize,
              int maxInputLength, int maxLabelLength, int alphabetSize, int blank, bool useCuda) {
  require_device(useCuda);
  raise_on(rnnt_hip_backward(emissions, predictions, egrads, pgrads, lngrads, alphas, logNorms,
                             labels, inputLengths, labelLengths, batchSize, maxInputLength,
                             maxLabelLength, alphabetSize, blank, nullptr));
}

void viterbi(const float* emissions, const float* predictions, const float* logNorms, int* labels,
             const int* inputLengths, const int* labelLengths, int batchSize, int maxInputLength,
             int maxLabelLength, int alphabetSize, int blank, bool useCuda) {
  require_device(useCuda);
  raise_on(rnnt_hip_viterbi(emissions, predictions, logNorms, labels, inputLengths, labelLengths,
                            batchSize, maxInputLength, maxLabelLength, alphabetSize, blank,
                            nullptr));
}
