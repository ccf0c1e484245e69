"""RNN-T loss for AMD MI355X (gfx950): drop-in for ``transducer.TransducerLoss``.

``TransducerLoss`` is looked up on first use, so that ``transducer_amd.build`` (which compiles
the native libraries) can be imported from a tree that does not hold them yet.  There is no
fallback: asking for ``TransducerLoss`` without the built libraries raises ImportError."""

__all__ = ["TransducerLoss"]


def __getattr__(name):
    if name == "TransducerLoss":
        from .torch_binding import TransducerLoss
        return TransducerLoss
    raise AttributeError("module %r has no attribute %r" % (__name__, name))
