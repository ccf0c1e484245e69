// pybind11 module `_transducer`: the three functions of the reference's module with the same
// keyword names (transducer/_transducer.cpp:41-54, 92-107, 137-148; note logNorms vs log_norms),
// pointers passed as Python ints, plus the fused entry points TransducerLoss uses, which take an
// explicit stream.  C++ exceptions from the layer below become ValueError / RuntimeError.
#include <pybind11/pybind11.h>

#include <cstdint>
#include <stdexcept>
#include <string>

#include "rnnt_hip.h"
#include "transducer.h"

namespace py = pybind11;
using namespace py::literals;
using ptr_t = std::uintptr_t;

namespace {

template <typename T>
T* as(ptr_t p) { return reinterpret_cast<T*>(p); }

void raise_on(int status) {
  if (status == RNNT_OK) return;
  const std::string msg = rnnt_hip_last_error();
  if (status == RNNT_HIP_FAILURE) throw std::runtime_error(msg);
  throw std::invalid_argument(msg);
}

}  // namespace

PYBIND11_MODULE(_transducer, m) {
  m.def("forward",
        [](ptr_t emissions, ptr_t predictions, ptr_t costs, ptr_t alphas, ptr_t logNorms,
           ptr_t labels, ptr_t input_lengths, ptr_t label_lengths, int batch_size,
           int max_input_length, int max_label_length, int alphabet_size, int blank,
           bool use_cuda) {
          forward(as<const float>(emissions), as<const float>(predictions), as<float>(costs),
                  as<float>(alphas), as<const float>(logNorms), as<const int>(labels),
                  as<const int>(input_lengths), as<const int>(label_lengths), batch_size,
                  max_input_length, max_label_length, alphabet_size, blank, use_cuda);
        },
        "emissions"_a, "predictions"_a, "costs"_a, "alphas"_a, "logNorms"_a, "labels"_a,
        "input_lengths"_a, "label_lengths"_a, "batch_size"_a, "max_input_length"_a,
        "max_label_length"_a, "alphabet_size"_a, "blank"_a, "use_cuda"_a);

  m.def("backward",
        [](ptr_t emissions, ptr_t predictions, ptr_t egrads, ptr_t pgrads, ptr_t lngrads,
           ptr_t alphas, ptr_t logNorms, ptr_t labels, ptr_t input_lengths, ptr_t label_lengths,
           int batch_size, int max_input_length, int max_label_length, int alphabet_size,
           int blank, bool use_cuda) {
          backward(as<const float>(emissions), as<const float>(predictions), as<float>(egrads),
                   as<float>(pgrads), as<float>(lngrads), as<const float>(alphas),
                   as<const float>(logNorms), as<const int>(labels), as<const int>(input_lengths),
                   as<const int>(label_lengths), batch_size, max_input_length, max_label_length,
                   alphabet_size, blank, use_cuda);
        },
        "emissions"_a, "predictions"_a, "egrads"_a, "pgrads"_a, "lngrads"_a, "alphas"_a,
        "logNorms"_a, "labels"_a, "input_lengths"_a, "label_lengths"_a, "batch_size"_a,
        "max_input_length"_a, "max_label_length"_a, "alphabet_size"_a, "blank"_a, "use_cuda"_a);

  m.def("viterbi",
        [](ptr_t emissions, ptr_t predictions, ptr_t log_norms, ptr_t labels, ptr_t input_lengths,
           ptr_t label_lengths, int batch_size, int max_input_length, int max_label_length,
           int alphabet_size, int blank, bool use_cuda) {
          viterbi(as<const float>(emissions), as<const float>(predictions),
                  as<const float>(log_norms), as<int>(labels), as<const int>(input_lengths),
                  as<const int>(label_lengths), batch_size, max_input_length, max_label_length,
                  alphabet_size, blank, use_cuda);
        },
        "emissions"_a, "predictions"_a, "log_norms"_a, "labels"_a, "input_lengths"_a,
        "label_lengths"_a, "batch_size"_a, "max_input_length"_a, "max_label_length"_a,
        "alphabet_size"_a, "blank"_a, "use_cuda"_a);

  // ---- beyond the reference's module: what its torch layer computed with bmm/exp/log ----
  m.def("log_norms",
        [](ptr_t emissions, ptr_t predictions, ptr_t log_norms, ptr_t input_lengths,
           ptr_t label_lengths, int batch_size, int max_input_length, int max_label_length,
           int alphabet_size, ptr_t stream) {
          raise_on(rnnt_hip_log_norms(as<const float>(emissions), as<const float>(predictions),
                                      as<float>(log_norms), as<const int>(input_lengths),
                                      as<const int>(label_lengths), batch_size, max_input_length,
                                      max_label_length, alphabet_size, as<void>(stream)));
        },
        "emissions"_a, "predictions"_a, "log_norms"_a, "input_lengths"_a, "label_lengths"_a,
        "batch_size"_a, "max_input_length"_a, "max_label_length"_a, "alphabet_size"_a,
        "stream"_a = 0);

  m.def("dense_grads",
        [](ptr_t emissions, ptr_t predictions, ptr_t egrads, ptr_t pgrads, ptr_t lngrads,
           ptr_t log_norms, ptr_t deltas, ptr_t input_lengths, ptr_t label_lengths,
           int batch_size, int max_input_length, int max_label_length, int alphabet_size,
           ptr_t stream) {
          raise_on(rnnt_hip_dense_grads(
              as<const float>(emissions), as<const float>(predictions), as<float>(egrads),
              as<float>(pgrads), as<const float>(lngrads), as<const float>(log_norms),
              as<const float>(deltas), as<const int>(input_lengths), as<const int>(label_lengths),
              batch_size, max_input_length, max_label_length, alphabet_size, as<void>(stream)));
        },
        "emissions"_a, "predictions"_a, "egrads"_a, "pgrads"_a, "lngrads"_a, "log_norms"_a,
        "deltas"_a, "input_lengths"_a, "label_lengths"_a, "batch_size"_a, "max_input_length"_a,
        "max_label_length"_a, "alphabet_size"_a, "stream"_a = 0);

  m.def("loss_workspace_bytes",
        [](int batch_size, int max_input_length, int max_label_length, int alphabet_size) {
          return rnnt_hip_loss_workspace_bytes(batch_size, max_input_length, max_label_length,
                                               alphabet_size);
        },
        "batch_size"_a, "max_input_length"_a, "max_label_length"_a, "alphabet_size"_a);

  m.def("loss_forward",
        [](ptr_t emissions, ptr_t predictions, ptr_t labels, ptr_t input_lengths,
           ptr_t label_lengths, ptr_t costs, ptr_t workspace, std::size_t workspace_bytes,
           int batch_size, int max_input_length, int max_label_length, int alphabet_size,
           int blank, ptr_t stream) {
          raise_on(rnnt_hip_loss_forward(
              as<const float>(emissions), as<const float>(predictions), as<const int>(labels),
              as<const int>(input_lengths), as<const int>(label_lengths), as<float>(costs),
              as<void>(workspace), workspace_bytes, batch_size, max_input_length,
              max_label_length, alphabet_size, blank, as<void>(stream)));
        },
        "emissions"_a, "predictions"_a, "labels"_a, "input_lengths"_a, "label_lengths"_a,
        "costs"_a, "workspace"_a, "workspace_bytes"_a, "batch_size"_a, "max_input_length"_a,
        "max_label_length"_a, "alphabet_size"_a, "blank"_a, "stream"_a = 0);

  m.def("loss_backward",
        [](ptr_t emissions, ptr_t predictions, ptr_t labels, ptr_t input_lengths,
           ptr_t label_lengths, ptr_t deltas, ptr_t egrads, ptr_t pgrads, ptr_t workspace,
           std::size_t workspace_bytes, int batch_size, int max_input_length,
           int max_label_length, int alphabet_size, int blank, ptr_t stream) {
          raise_on(rnnt_hip_loss_backward(
              as<const float>(emissions), as<const float>(predictions), as<const int>(labels),
              as<const int>(input_lengths), as<const int>(label_lengths), as<const float>(deltas),
              as<float>(egrads), as<float>(pgrads), as<void>(workspace), workspace_bytes,
              batch_size, max_input_length, max_label_length, alphabet_size, blank,
              as<void>(stream)));
        },
        "emissions"_a, "predictions"_a, "labels"_a, "input_lengths"_a, "label_lengths"_a,
        "deltas"_a, "egrads"_a, "pgrads"_a, "workspace"_a, "workspace_bytes"_a, "batch_size"_a,
        "max_input_length"_a, "max_label_length"_a, "alphabet_size"_a, "blank"_a, "stream"_a = 0);

  // 16-bit scores and gradients, bf16 and fp16 (no counterpart in the reference, which takes
  // float32 only)
  m.def("loss_forward_bf16",
        [](ptr_t emissions, ptr_t predictions, ptr_t labels, ptr_t input_lengths,
           ptr_t label_lengths, ptr_t costs, ptr_t workspace, std::size_t workspace_bytes,
           int batch_size, int max_input_length, int max_label_length, int alphabet_size,
           int blank, ptr_t stream) {
          raise_on(rnnt_hip_loss_forward_bf16(
              as<const uint16_t>(emissions), as<const uint16_t>(predictions),
              as<const int>(labels), as<const int>(input_lengths), as<const int>(label_lengths),
              as<float>(costs), as<void>(workspace), workspace_bytes, batch_size,
              max_input_length, max_label_length, alphabet_size, blank, as<void>(stream)));
        },
        "emissions"_a, "predictions"_a, "labels"_a, "input_lengths"_a, "label_lengths"_a,
        "costs"_a, "workspace"_a, "workspace_bytes"_a, "batch_size"_a, "max_input_length"_a,
        "max_label_length"_a, "alphabet_size"_a, "blank"_a, "stream"_a = 0);

  m.def("loss_forward_f16",
        [](ptr_t emissions, ptr_t predictions, ptr_t labels, ptr_t input_lengths,
           ptr_t label_lengths, ptr_t costs, ptr_t workspace, std::size_t workspace_bytes,
           int batch_size, int max_input_length, int max_label_length, int alphabet_size,
           int blank, ptr_t stream) {
          raise_on(rnnt_hip_loss_forward_f16(
              as<const uint16_t>(emissions), as<const uint16_t>(predictions),
              as<const int>(labels), as<const int>(input_lengths), as<const int>(label_lengths),
              as<float>(costs), as<void>(workspace), workspace_bytes, batch_size,
              max_input_length, max_label_length, alphabet_size, blank, as<void>(stream)));
        },
        "emissions"_a, "predictions"_a, "labels"_a, "input_lengths"_a, "label_lengths"_a,
        "costs"_a, "workspace"_a, "workspace_bytes"_a, "batch_size"_a, "max_input_length"_a,
        "max_label_length"_a, "alphabet_size"_a, "blank"_a, "stream"_a = 0);

  m.def("loss_backward_bf16",
        [](ptr_t emissions, ptr_t predictions, ptr_t labels, ptr_t input_lengths,
           ptr_t label_lengths, ptr_t deltas, ptr_t egrads, ptr_t pgrads, ptr_t workspace,
           std::size_t workspace_bytes, int batch_size, int max_input_length,
           int max_label_length, int alphabet_size, int blank, ptr_t stream) {
          raise_on(rnnt_hip_loss_backward_bf16(
              as<const uint16_t>(emissions), as<const uint16_t>(predictions),
              as<const int>(labels), as<const int>(input_lengths), as<const int>(label_lengths),
              as<const float>(deltas), as<uint16_t>(egrads), as<uint16_t>(pgrads),
              as<void>(workspace), workspace_bytes, batch_size, max_input_length,
              max_label_length, alphabet_size, blank, as<void>(stream)));
        },
        "emissions"_a, "predictions"_a, "labels"_a, "input_lengths"_a, "label_lengths"_a,
        "deltas"_a, "egrads"_a, "pgrads"_a, "workspace"_a, "workspace_bytes"_a, "batch_size"_a,
        "max_input_length"_a, "max_label_length"_a, "alphabet_size"_a, "blank"_a, "stream"_a = 0);

  m.def("loss_backward_f16",
        [](ptr_t emissions, ptr_t predictions, ptr_t labels, ptr_t input_lengths,
           ptr_t label_lengths, ptr_t deltas, ptr_t egrads, ptr_t pgrads, ptr_t workspace,
           std::size_t workspace_bytes, int batch_size, int max_input_length,
           int max_label_length, int alphabet_size, int blank, ptr_t stream) {
          raise_on(rnnt_hip_loss_backward_f16(
              as<const uint16_t>(emissions), as<const uint16_t>(predictions),
              as<const int>(labels), as<const int>(input_lengths), as<const int>(label_lengths),
              as<const float>(deltas), as<uint16_t>(egrads), as<uint16_t>(pgrads),
              as<void>(workspace), workspace_bytes, batch_size, max_input_length,
              max_label_length, alphabet_size, blank, as<void>(stream)));
        },
        "emissions"_a, "predictions"_a, "labels"_a, "input_lengths"_a, "label_lengths"_a,
        "deltas"_a, "egrads"_a, "pgrads"_a, "workspace"_a, "workspace_bytes"_a, "batch_size"_a,
        "max_input_length"_a, "max_label_length"_a, "alphabet_size"_a, "blank"_a, "stream"_a = 0);

  m.def("viterbi_decode",
        [](ptr_t emissions, ptr_t predictions, ptr_t input_lengths, ptr_t label_lengths,
           ptr_t labels, int batch_size, int max_input_length, int max_label_length,
           int alphabet_size, int blank, ptr_t stream) {
          raise_on(rnnt_hip_viterbi_decode(
              as<const float>(emissions), as<const float>(predictions),
              as<const int>(input_lengths), as<const int>(label_lengths), as<int>(labels),
              batch_size, max_input_length, max_label_length, alphabet_size, blank,
              as<void>(stream)));
        },
        "emissions"_a, "predictions"_a, "input_lengths"_a, "label_lengths"_a, "labels"_a,
        "batch_size"_a, "max_input_length"_a, "max_label_length"_a, "alphabet_size"_a, "blank"_a,
        "stream"_a = 0);

  m.def("viterbi_decode_bf16",
        [](ptr_t emissions, ptr_t predictions, ptr_t input_lengths, ptr_t label_lengths,
           ptr_t labels, int batch_size, int max_input_length, int max_label_length,
           int alphabet_size, int blank, ptr_t stream) {
          raise_on(rnnt_hip_viterbi_decode_bf16(
              as<const uint16_t>(emissions), as<const uint16_t>(predictions),
              as<const int>(input_lengths), as<const int>(label_lengths), as<int>(labels),
              batch_size, max_input_length, max_label_length, alphabet_size, blank,
              as<void>(stream)));
        },
        "emissions"_a, "predictions"_a, "input_lengths"_a, "label_lengths"_a, "labels"_a,
        "batch_size"_a, "max_input_length"_a, "max_label_length"_a, "alphabet_size"_a, "blank"_a,
        "stream"_a = 0);

  m.def("viterbi_decode_f16",
        [](ptr_t emissions, ptr_t predictions, ptr_t input_lengths, ptr_t label_lengths,
           ptr_t labels, int batch_size, int max_input_length, int max_label_length,
           int alphabet_size, int blank, ptr_t stream) {
          raise_on(rnnt_hip_viterbi_decode_f16(
              as<const uint16_t>(emissions), as<const uint16_t>(predictions),
              as<const int>(input_lengths), as<const int>(label_lengths), as<int>(labels),
              batch_size, max_input_length, max_label_length, alphabet_size, blank,
              as<void>(stream)));
        },
        "emissions"_a, "predictions"_a, "input_lengths"_a, "label_lengths"_a, "labels"_a,
        "batch_size"_a, "max_input_length"_a, "max_label_length"_a, "alphabet_size"_a, "blank"_a,
        "stream"_a = 0);

#ifdef VERSION_INFO
  m.attr("__version__") = VERSION_INFO;
#else
  m.attr("__version__") = "dev";
#endif
}
