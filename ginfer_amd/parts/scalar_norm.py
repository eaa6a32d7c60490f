"""RMS norm with one gain for all coordinates."""
from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import Part
from .registry import register_norm


@register_norm("scalar_rmsnorm")
class ScalarRMSNorm(Part):
    """y = g * x / sqrt(mean(x^2) + eps), g a single number (the tensor is named as the part itself: its local name is
    empty).  Computed in 32-bit.  Two uses: `forward`, the usual face of a norm (adds a pending delta into the residual
    stream, returns the normalised rows, all or the listed ones), and `add_normed`, for blocks that norm a sublayer's
    OUTPUT: residual += norm(y)."""

    capturable = True
    accepts_partial_sums = False
    foldable = False         # the products around it cannot fold it: it does not sit before a product

    def __init__(self, size, eps, dtype, device):
        self.size, self.eps, self.dtype, self.device = int(size), float(eps), dtype, device
        self.weight = None

    def weight_specs(self):
        return {"": WeightSpec((), init="one_plus_normal", keep_32bit=True)}

    def bind_weights(self, tensors):
        self.weight = tensors[""].float().reshape(1).contiguous()

    def kernel_modules(self):
        return ["scalar_norm"]

    def forward(self, residual, delta=None, rows=None):
        if delta is not None:
            if rows is None:
                residual.add_(delta)
            else:
                residual = residual + delta
        return ops.scalar_rmsnorm_rows(residual, self.weight, self.eps, self.dtype, rows=rows)

    def add_normed(self, residual, y, copy=False):
        """residual += norm(y) in place.  With copy: the new residual in the compute dtype (for the product that reads it
        next); in 32-bit that is the residual itself."""
        return ops.add_scalar_rmsnorm(residual, y, self.weight, self.eps, copy=copy)
