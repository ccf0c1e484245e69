"""PyTorch front end: ``TransducerLoss()(emissions, predictions, labels, input_lengths,
label_lengths)`` and ``criterion.viterbi(...)`` with the signatures, checks and error messages of
the reference's ``transducer/torch_binding.py``.

Where the reference computes the log-normaliser and the dense gradient parts with
``max/exp/bmm/log`` on [B,T,V]-sized temporaries (``torch_binding.py:35-40, 85-89``), this module
makes two calls into the HIP library, which keeps only O(B*T*U) state between forward and
backward.  torch is used for tensors, the autograd hook and the current stream, nothing else.
All tensors must live on one HIP device (``tensor.is_cuda``); there is no CPU backend.
"""
import torch

from . import _transducer


class DeviceManager(object):
    """``with DeviceManager(device):`` runs its body with `device` as torch's current HIP device
    and puts the previous one back afterwards, as the reference brackets every library call
    (torch_binding.py:7-20): the library works on the current device's pointers."""

    def __init__(self, device):
        self.device = device
        self.is_cuda = device.type == "cuda"
        self._previous = None

    def __enter__(self):
        if not self.is_cuda:
            return self
        self._previous = torch.cuda.current_device()
        torch.cuda.set_device(self.device)
        return self

    def __exit__(self, *exc_info):
        if self._previous is not None:
            torch.cuda.set_device(self._previous)
            self._previous = None
        return False


def _require_device(tensor):
    if not tensor.is_cuda:
        # same exception the C++ interface raises for host pointers
        raise ValueError("Transducer not built with the CPU backend.")


# entry-point suffix per 16-bit score type
_SUFFIX = {torch.bfloat16: "_bf16", torch.float16: "_f16"}


def _check_blank(blank, vocabulary):
    """The reference indexes score rows with `blank` unchecked; an index outside the vocabulary
    would read and write past every row, so it is refused (the library refuses it as well)."""
    if not 0 <= blank < vocabulary:
        raise ValueError("blank must lie in [0, {}), got {}".format(vocabulary, blank))


def _stream(device):
    return torch.cuda.current_stream(device).cuda_stream


class Transducer(torch.autograd.Function):
    """costs[B] = -log p(labels | emissions, predictions); reference: torch_binding.py:23-90."""

    @staticmethod
    def forward(ctx, emissions, predictions, labels, input_lengths, label_lengths, blank=0,
                low_precision=()):
        suffix = _SUFFIX[emissions.dtype] if emissions.dtype in low_precision else ""
        certify_inputs(emissions, predictions, labels, input_lengths, label_lengths,
                       score_dtype=emissions.dtype if suffix else torch.float32)
        _require_device(emissions)
        _check_blank(blank, emissions.shape[2])
        device = emissions.device
        # the library reads raw pointers: dense row-major storage is required
        emissions = emissions.contiguous()
        predictions = predictions.contiguous()
        B, T, V = emissions.shape
        U = predictions.shape[1]
        costs = torch.empty(size=(B,), device=device, dtype=torch.float32)
        nbytes = _transducer.loss_workspace_bytes(B, T, U, V)
        workspace = torch.empty(size=(nbytes,), device=device, dtype=torch.uint8)
        with DeviceManager(device):
            getattr(_transducer, "loss_forward" + suffix)(
                emissions.data_ptr(), predictions.data_ptr(), labels.data_ptr(),
                input_lengths.data_ptr(), label_lengths.data_ptr(), costs.data_ptr(),
                workspace.data_ptr(), nbytes, B, T, U, V, blank, _stream(device))
        ctx.save_for_backward(
            emissions, predictions, labels, input_lengths, label_lengths, workspace)
        ctx.blank = blank
        ctx.suffix = suffix
        return costs

    @staticmethod
    def backward(ctx, deltas):
        emissions, predictions, labels, input_lengths, label_lengths, workspace = \
            ctx.saved_tensors
        device = emissions.device
        B, T, V = emissions.shape
        U = predictions.shape[1]
        deltas = deltas.contiguous()
        egrads = torch.empty(size=(B, T, V), device=device, dtype=emissions.dtype)
        pgrads = torch.empty(size=(B, U, V), device=device, dtype=emissions.dtype)
        with DeviceManager(device):
            getattr(_transducer, "loss_backward" + ctx.suffix)(
                emissions.data_ptr(), predictions.data_ptr(), labels.data_ptr(),
                input_lengths.data_ptr(), label_lengths.data_ptr(), deltas.data_ptr(),
                egrads.data_ptr(), pgrads.data_ptr(), workspace.data_ptr(), workspace.numel(),
                B, T, U, V, ctx.blank, _stream(device))
        return egrads, pgrads, None, None, None, None, None


class TransducerLoss(torch.nn.Module):
    """RNN transducer loss: per-utterance negative log-likelihood of the label sequence, summed
    over all alignments of the joint scores ``emissions[b,t,:] + predictions[b,u,:]``.

    Same constructor and call signature as the reference's module (torch_binding.py:93-128);
    every tensor has to sit on one HIP device.

    blank: id of the blank symbol (0 unless given).
    allow_bf16, allow_fp16: when True, ``torch.bfloat16`` / ``torch.float16`` emissions and
        predictions (both of the same type) are accepted as well; costs are float32 and the
        gradients come back in the scores' type.  The reference raises ``TypeError`` for
        anything but float32, and so does this module unless a flag is set.  The loss takes at
        most 1025 label positions in these types (any vocabulary size).
    """

    def __init__(self, blank=0, allow_bf16=False, allow_fp16=False):
        super(TransducerLoss, self).__init__()
        self.blank = blank
        self.allow_bf16 = allow_bf16
        self.allow_fp16 = allow_fp16

    @property
    def low_precision(self):
        """Score types accepted besides float32."""
        return tuple(t for t, on in ((torch.bfloat16, self.allow_bf16),
                                     (torch.float16, self.allow_fp16)) if on)

    def forward(self, emissions, predictions, labels, input_lengths, label_lengths):
        """costs[B] (float32) for a padded batch.

        emissions:      float32 [B, T, V]     encoder-side scores, unnormalised
        predictions:    float32 [B, U + 1, V] label-side scores, unnormalised (row u is used
                                              after u labels have been emitted)
        labels:         int32   [B, U]        targets, padded to the longest one
        input_lengths:  int32   [B]           frames in use per utterance
        label_lengths:  int32   [B]           labels in use per utterance

        Differentiable with respect to emissions and predictions (once)."""
        return Transducer.apply(
            emissions, predictions, labels, input_lengths, label_lengths, self.blank,
            self.low_precision)

    @torch.no_grad()
    def viterbi(self, emissions, predictions, input_lengths, label_lengths):
        """Best alignment with the prediction rows forced and the number of labels per utterance
        given; returns the labels on it as int32 [B, U] (reference: torch_binding.py:130-177).
        Entries past an utterance's label length are unwritten padding."""
        device = emissions.device
        B, T, V = emissions.shape
        U = predictions.shape[1]
        labels = torch.empty(size=(B, U - 1), device=device, dtype=torch.int32)
        suffix = _SUFFIX[emissions.dtype] if emissions.dtype in self.low_precision else ""
        certify_inputs(emissions, predictions, labels, input_lengths, label_lengths,
                       score_dtype=emissions.dtype if suffix else torch.float32)
        _require_device(emissions)
        _check_blank(self.blank, V)
        emissions = emissions.contiguous()
        predictions = predictions.contiguous()
        with DeviceManager(device):
            getattr(_transducer, "viterbi_decode" + suffix)(
                emissions.data_ptr(), predictions.data_ptr(), input_lengths.data_ptr(),
                label_lengths.data_ptr(), labels.data_ptr(), B, T, U, V, self.blank,
                _stream(device))
        return labels


def certify_inputs(emissions, predictions, labels, input_lengths, label_lengths,
                   score_dtype=torch.float32):
    """Argument validation with the reference's exception types, message texts and ORDER of
    checks (torch_binding.py:180-229), so a caller sees the same error for the same mistake:
    element types, then dense storage of the integer arrays, then sizes that must agree, then
    ranks, then the padded extents against the longest utterance."""
    named = (("emissions", emissions, score_dtype, 3), ("predictions", predictions, score_dtype, 3),
             ("labels", labels, torch.int32, 2), ("input_lengths", input_lengths, torch.int32, 1),
             ("label_lengths", label_lengths, torch.int32, 1))
    for name, tensor, dtype, _ in named:
        if tensor.dtype is not dtype:
            raise TypeError("{} must be {}".format(name, dtype))
    # (the reference reports input_lengths under the name "lengths" here)
    for shown, tensor in (("labels", labels), ("label_lengths", label_lengths),
                          ("lengths", input_lengths)):
        if not tensor.is_contiguous():
            raise ValueError("{} must be contiguous".format(shown))
    # evaluated one after the other: an array of the wrong rank fails in the first relation that
    # indexes a missing axis, before the rank checks below, exactly as it does upstream
    batch = emissions.shape[0]
    agreements = (
        (lambda: emissions.shape[2] == predictions.shape[2], "vocab size mismatch."),
        (lambda: input_lengths.shape[0] == batch, "must have a length per example."),
        (lambda: label_lengths.shape[0] == batch, "must have a label length per example."),
        (lambda: labels.shape[0] == batch, "must have a label per example."),
        (lambda: labels.shape[1] == predictions.shape[1] - 1,
         "labels must be padded to maximum label length."),
    )
    for holds, message in agreements:
        if not holds():
            raise ValueError(message)
    for name, tensor, _, rank in named:
        if tensor.dim() != rank:
            raise ValueError("{} must be {}D".format(name, rank))
    if emissions.shape[1] < int(input_lengths.max()):
        raise ValueError("Input length mismatch")
    if predictions.shape[1] < int(label_lengths.max()) + 1:
        raise ValueError("Output length mismatch")
