// C++ interface of the RNN-T loss library -- the same three free functions, with the same
// argument order and C++ linkage, as awni/transducer's transducer/transducer.h:3-49, so code
// written against that header links against libtransducer.so unchanged.
//
// Backend selection follows the reference's last argument:
//   useCuda == true   every pointer is a device pointer on the current HIP device ("cuda" is
//                     the name PyTorch-ROCm gives HIP devices); work is enqueued on the null
//                     stream and the call returns without waiting, as cuda::forward etc. do
//                     (transducer/transducer_cuda.cu:280-388).
//   useCuda == false  host pointers.  This build carries no CPU backend: the call throws
//                     std::invalid_argument("Transducer not built with the CPU backend."),
//                     mirroring what the reference does for a backend that was compiled out
//                     (transducer/transducer.cpp:41,97,147).
//
// maxLabelLength is the second dimension of `predictions`, i.e. the longest label + 1.
// Failures of the HIP runtime surface as std::runtime_error("[file:line] HIP error: ..."),
// bad arguments as std::invalid_argument.
#pragma once

// alpha recursion.  in: emissions [B,T,V], predictions [B,U,V], logNorms [B,T,U],
// labels [B,U-1], inputLengths/labelLengths [B].  out: costs [B], alphas [B,T,U].
void forward(const float* emissions, const float* predictions, float* costs, float* alphas,
             const float* logNorms, const int* labels, const int* inputLengths,
             const int* labelLengths, int batchSize, int maxInputLength, int maxLabelLength,
             int alphabetSize, int blank, bool useCuda);

// dalpha recursion.  out (zero-filled by the library first): egrads [B,T,V] and pgrads [B,U,V]
// holding the sparse blank/label terms, lngrads [B,T,U] = d cost / d logNorms.
void backward(const float* emissions, const float* predictions, float* egrads, float* pgrads,
              float* lngrads, const float* alphas, const float* logNorms, const int* labels,
              const int* inputLengths, const int* labelLengths, int batchSize,
              int maxInputLength, int maxLabelLength, int alphabetSize, int blank, bool useCuda);

// best path of the given lengths.  out: labels [B,U-1], first labelLengths[b] entries per row.
void viterbi(const float* emissions, const float* predictions, const float* logNorms, int* labels,
             const int* inputLengths, const int* labelLengths, int batchSize, int maxInputLength,
             int maxLabelLength, int alphabetSize, int blank, bool useCuda);
