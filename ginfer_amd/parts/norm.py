"""RMSNorm fused with the residual add that precedes it."""
import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import Part
from .registry import register_norm


@register_norm("rmsnorm")
class RMSNorm(Part):
    """y = (h * g) / sqrt(mean(h^2) + eps) with h = residual + delta; plain gain, no bias, no mean
    subtraction (ginfer/core/op/kernels/cuda/rmsnorm_kernel.cu:27-66, ginfer/core/layer/rmsnorm.cc:6-22).
    gain_offset: a checkpoint that stores its gains around zero says 1.0 here, and g = offset + stored; the sum is
    taken once, in 32-bit, when the weights are bound.  weight_name: the tensor's name inside the part ("" where the
    checkpoint names it as the part itself)."""

    capturable = True
    accepts_partial_sums = True

    def __init__(self, size, eps, dtype, device, gain_offset=0.0, weight_name="weight"):
        self.size, self.eps, self.dtype, self.device = int(size), float(eps), dtype, device
        self.gain_offset, self.weight_name = float(gain_offset), str(weight_name)
        # a plain gain over the root mean square in the compute dtype: the products around it can fold it
        self.foldable = self.gain_offset == 0.0
        self.weight = None

    def weight_specs(self):
        return {self.weight_name: WeightSpec((self.size,), init="normal" if self.gain_offset else "one_plus_normal",
                                             keep_32bit=True)}

    def bind_weights(self, tensors):
        w = tensors[self.weight_name]
        self.weight = (w.float() + self.gain_offset).contiguous() if self.gain_offset else w

    def kernel_modules(self):
        return ["norm"]

    def forward(self, residual, delta=None, rows=None):
        return ops.add_rmsnorm(residual, delta, self.weight, self.eps, self.dtype, rows=rows)


@register_norm("scaled_output_rmsnorm")
class ScaledOutputRMSNorm(Part):
    """A norm on a sublayer's OUTPUT, with a factor per channel behind it (a layer scale):
    residual += s * (offset + g) * y / sqrt(mean(y^2) + eps).  Computed in 32-bit.  `add_normed(residual, y, then)`
    does that in place; with `then`, the norm in front of the sublayer that runs next (a plain gain: `weight`, `eps`),
    the same launch also returns that norm's rows of the new residual.  gain_name, scale_name: the two tensors' names
    inside the part (scale_name None: no such factor)."""

    capturable = True
    accepts_partial_sums = True      # add_normed takes float32 [parts, T, H] and adds the parts up in order
    foldable = False

    def __init__(self, size, eps, dtype, device, gain_offset=0.0, gain_name="weight", scale_name="scale"):
        self.size, self.eps, self.dtype, self.device = int(size), float(eps), dtype, device
        self.gain_offset, self.gain_name = float(gain_offset), str(gain_name)
        self.scale_name = None if scale_name is None else str(scale_name)
        self.weight = self.scale = None

    def weight_specs(self):
        specs = {self.gain_name: WeightSpec((self.size,), init="normal" if self.gain_offset else "one_plus_normal",
                                            keep_32bit=True)}
        if self.scale_name is not None:
            specs[self.scale_name] = WeightSpec((self.size,), init="one_plus_normal", std=0.2, keep_32bit=True)
        return specs

    def bind_weights(self, tensors):
        self.weight = (tensors[self.gain_name].float() + self.gain_offset).contiguous()
        self.scale = tensors[self.scale_name].float().contiguous() if self.scale_name is not None else None

    def kernel_modules(self):
        return ["output_norm"]

    def add_normed(self, residual, y, then=None):
        if then is None:
            return ops.output_norm_add(residual, y, self.weight, self.scale, self.eps)
        gain = then.weight if then.weight.dtype == torch.float32 else then.weight.float()
        return ops.output_norm_add(residual, y, self.weight, self.scale, self.eps, gain, then.eps, then.dtype)
