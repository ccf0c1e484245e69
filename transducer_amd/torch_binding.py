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
    """Makes the tensors' device current for the duration of a library call
    (reference: torch_binding.py:7-20)."""

    def __init__(self, device):
        self.device = device
        self.is_cuda = device.type == "cuda"

    def __enter__(self):
        if self.is_cuda:
            self.old_device = torch.cuda.current_device()
            torch.cuda.set_device(self.device)

    def __exit__(self, exc_type, exc_value, traceback):
        if self.is_cuda:
            torch.cuda.set_device(self.old_device)


def _require_device(tensor):
    if not tensor.is_cuda:
        # same exception the C++ interface raises for host pointers
        raise ValueError("Transducer not built with the CPU backend.")


def _stream(device):
    return torch.cuda.current_stream(device).cuda_stream


class Transducer(torch.autograd.Function):
    """costs[B] = -log p(labels | emissions, predictions); reference: torch_binding.py:23-90."""

    @staticmethod
    def forward(ctx, emissions, predictions, labels, input_lengths, label_lengths, blank=0,
                allow_bf16=False):
        bf16 = allow_bf16 and emissions.dtype is torch.bfloat16
        certify_inputs(emissions, predictions, labels, input_lengths, label_lengths,
                       score_dtype=torch.bfloat16 if bf16 else torch.float32)
        _require_device(emissions)
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
            (_transducer.loss_forward_bf16 if bf16 else _transducer.loss_forward)(
                emissions.data_ptr(), predictions.data_ptr(), labels.data_ptr(),
                input_lengths.data_ptr(), label_lengths.data_ptr(), costs.data_ptr(),
                workspace.data_ptr(), nbytes, B, T, U, V, blank, _stream(device))
        ctx.save_for_backward(
            emissions, predictions, labels, input_lengths, label_lengths, workspace)
        ctx.blank = blank
        ctx.bf16 = bf16
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
            (_transducer.loss_backward_bf16 if ctx.bf16 else _transducer.loss_backward)(
                emissions.data_ptr(), predictions.data_ptr(), labels.data_ptr(),
                input_lengths.data_ptr(), label_lengths.data_ptr(), deltas.data_ptr(),
                egrads.data_ptr(), pgrads.data_ptr(), workspace.data_ptr(), workspace.numel(),
                B, T, U, V, ctx.blank, _stream(device))
        return egrads, pgrads, None, None, None, None, None


class TransducerLoss(torch.nn.Module):
    """
    The RNN-T loss function.

    All input tensors must be on the same HIP device.

    Arguments:
        blank (int, optional): Integer id of blank label (default is 0).
        allow_bf16 (bool, optional): also accept ``torch.bfloat16`` emissions and predictions
            (both), returning float32 costs and bfloat16 gradients.  Not in the reference, which
            raises ``TypeError`` for anything but float32 -- and so does this module by default.
            Needs a vocabulary that is a multiple of 8 and at most 112 label positions.
    """

    def __init__(self, blank=0, allow_bf16=False):
        super(TransducerLoss, self).__init__()
        self.blank = blank
        self.allow_bf16 = allow_bf16

    def forward(self, emissions, predictions, labels, input_lengths, label_lengths):
        """
        Arguments:
          emissions (FloatTensor): unnormalized emission scores,
            (minibatch, input length, vocab size).
          predictions (FloatTensor): unnormalized prediction scores,
            (minibatch, output length + 1, vocab size).
          labels (IntTensor): (minibatch, output length), padded to the longest label.
          input_lengths (IntTensor): (minibatch,) input length of each example.
          label_lengths (IntTensor): (minibatch,) label length of each example.

        Returns:
          costs (FloatTensor): (minibatch,) negative log-likelihood of each example.
        """
        return Transducer.apply(
            emissions, predictions, labels, input_lengths, label_lengths, self.blank,
            self.allow_bf16)

    @torch.no_grad()
    def viterbi(self, emissions, predictions, input_lengths, label_lengths):
        """
        Viterbi decoding of the RNN-T graph with teacher-forced predictions and given output
        lengths (reference: torch_binding.py:130-177).

        Returns:
          labels (IntTensor): (minibatch, output length); entries past an example's label
          length are arbitrary padding.
        """
        device = emissions.device
        B, T, V = emissions.shape
        U = predictions.shape[1]
        labels = torch.empty(size=(B, U - 1), device=device, dtype=torch.int32)
        bf16 = self.allow_bf16 and emissions.dtype is torch.bfloat16
        certify_inputs(emissions, predictions, labels, input_lengths, label_lengths,
                       score_dtype=torch.bfloat16 if bf16 else torch.float32)
        _require_device(emissions)
        emissions = emissions.contiguous()
        predictions = predictions.contiguous()
        with DeviceManager(device):
            (_transducer.viterbi_decode_bf16 if bf16 else _transducer.viterbi_decode)(
                emissions.data_ptr(), predictions.data_ptr(), input_lengths.data_ptr(),
                label_lengths.data_ptr(), labels.data_ptr(), B, T, U, V, self.blank,
                _stream(device))
        return labels


def check_type(var, t, name):
    if var.dtype is not t:
        raise TypeError("{} must be {}".format(name, t))


def check_contiguous(var, name):
    if not var.is_contiguous():
        raise ValueError("{} must be contiguous".format(name))


def check_dim(var, dim, name):
    if len(var.shape) != dim:
        raise ValueError("{} must be {}D".format(name, dim))


def certify_inputs(emissions, predictions, labels, input_lengths, label_lengths,
                   score_dtype=torch.float32):
    """Same checks, order and messages as the reference (torch_binding.py:195-229)."""
    check_type(emissions, score_dtype, "emissions")
    check_type(predictions, score_dtype, "predictions")
    check_type(labels, torch.int32, "labels")
    check_type(input_lengths, torch.int32, "input_lengths")
    check_type(label_lengths, torch.int32, "label_lengths")
    check_contiguous(labels, "labels")
    check_contiguous(label_lengths, "label_lengths")
    check_contiguous(input_lengths, "lengths")

    batchSize = emissions.shape[0]
    if emissions.shape[2] != predictions.shape[2]:
        raise ValueError("vocab size mismatch.")
    if input_lengths.shape[0] != batchSize:
        raise ValueError("must have a length per example.")
    if label_lengths.shape[0] != batchSize:
        raise ValueError("must have a label length per example.")
    if labels.shape[0] != batchSize:
        raise ValueError("must have a label per example.")
    if labels.shape[1] != (predictions.shape[1] - 1):
        raise ValueError("labels must be padded to maximum label length.")

    check_dim(emissions, 3, "emissions")
    check_dim(predictions, 3, "predictions")
    check_dim(labels, 2, "labels")
    check_dim(input_lengths, 1, "input_lengths")
    check_dim(label_lengths, 1, "label_lengths")
    max_T = torch.max(input_lengths)
    max_U = torch.max(label_lengths)
    T = emissions.shape[1]
    U = predictions.shape[1]
    if T < max_T:
        raise ValueError("Input length mismatch")
    if U < max_U + 1:
        raise ValueError("Output length mismatch")
