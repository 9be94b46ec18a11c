"""Quantizer interface shared by every quantizer module (the contract of the reference's
src/models/quantization/quantizers/base.py:6-24): calling the module returns the pseudo-quantized tensor,
``re_randomize()`` draws a fresh random rotation where the quantizer has one, and ``bits`` / ``n_levels``
describe the grid."""
import torch.nn as nn


class BaseQuantizer(nn.Module):
    """Abstract quantizer: subclasses implement ``forward(x)``; a quantizer without randomness inherits the
    no-op ``re_randomize``."""

    def __init__(self, bits=4):
        super().__init__()
        self.bits = bits

    @property
    def n_levels(self):
        return 2 ** self.bits

    def forward(self, x):
        raise NotImplementedError(f"{type(self).__name__} does not implement forward()")

    def re_randomize(self):
        return None


class NoQuantizer(BaseQuantizer):
    """Identity: the tensor passes through untouched (reported as a 16-bit grid).  Accepts and ignores any
    keyword arguments so that registry-driven constructors can pass a kwargs dict."""

    def __init__(self, **_ignored):
        super().__init__(bits=16)

    def forward(self, x):
        return x
