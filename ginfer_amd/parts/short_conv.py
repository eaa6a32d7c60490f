"""A short causal convolution over time on what a mixer reads."""
import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import Part, StateSpec
from .registry import register_convolution


@register_convolution("short_causal")
class ShortCausalConvolution(Part):
    """h_t = x_t + sum_j w[:, j] * x_(t - taps + 1 + j) on each channel of the 32-bit stream, zeros before the sequence's
    start, no bias (`residual=False`: the sum alone).  The last taps - 1 inputs of a request are its state (32-bit, one
    slot per request); a request's first tokens start from zeros.  The result comes in the compute dtype, which is what
    the mixer's products read.  The weight tensor [width, taps] is named as the part itself."""

    capturable = True

    def __init__(self, width, taps, dtype, device, residual=True):
        if not 1 <= int(taps) <= ops.SHORT_CONV_MAX_TAPS:
            raise ValueError("the short convolution takes 1 to %d taps, got %r" % (ops.SHORT_CONV_MAX_TAPS, taps))
        self.width, self.taps, self.residual = int(width), int(taps), bool(residual)
        self.dtype, self.device = dtype, device
        self.weight = None

    def cache_spec(self):
        return StateSpec((self.taps - 1, self.width), torch.float32) if self.taps > 1 else None

    def weight_specs(self):
        return {"": WeightSpec((self.width, self.taps), std=0.2)}

    def bind_weights(self, tensors):
        self.weight = tensors[""].float().contiguous()

    def kernel_modules(self):
        return ["short_conv"]

    def forward(self, x, step, cache):
        """x float32 [T, width]; cache: the StateView of this run (None for one tap)."""
        if cache is None:
            return ops.short_conv(x, self.weight, None, None, step, self.dtype, add_input=self.residual)
        return ops.short_conv(x, self.weight, cache.state, cache.slots, step, self.dtype, add_input=self.residual,
                              update=cache.owner)
