"""RNN-T loss for AMD MI355X (gfx950): drop-in for ``transducer.TransducerLoss``."""
from .torch_binding import TransducerLoss  # noqa: F401

__all__ = ["TransducerLoss"]
