"""What happens to the residual stream where a run of layers is entered again."""
import torch

from ..weights.loader import WeightSpec
from .base import Part
from .linear import linear
from .registry import register_reentry


@register_reentry("concat_projection")
class ConcatProjectionReentry(Part):
    """Before pass t of a group of layers that runs several times: x <- W [x; x0] + s_t, with x0 the embedding's output,
    W [H, 2H] (x's half first) and s [passes, H] one vector per pass.  The product may run in the compute dtype; the
    sum and the new stream are 32-bit.  W is split into its halves when it is bound: the half that reads x0 is
    multiplied once a step (`prepare`), not once a pass.  Tensors: `in` and `step` unless named otherwise."""

    capturable = True

    def __init__(self, hidden_size, passes, dtype, device, weight_name="in", step_name="step"):
        self.hidden_size, self.passes = int(hidden_size), int(passes)
        self.weight_name, self.step_name = str(weight_name), str(step_name)
        self.dtype, self.device = dtype, device
        self.w_stream = self.w_first = self.steps = None

    def weight_specs(self):
        H = self.hidden_size
        return {self.weight_name: WeightSpec((H, 2 * H)), self.step_name: WeightSpec((self.passes, H), keep_32bit=True)}

    def bind_weights(self, t):
        w = t[self.weight_name]
        H = self.hidden_size
        self.w_stream, self.w_first = w[:, :H].contiguous(), w[:, H:].contiguous()
        self.steps = t[self.step_name].float().contiguous()

    def kernel_modules(self):
        return ["gemm"] + (["gemm_skinny"] if self.dtype == torch.bfloat16 else [])

    def prepare(self, first):
        """first: the embedding's output, float32 [T, H] -> what every pass of the step adds: W_first x0, 32-bit."""
        x0 = first if self.dtype == torch.float32 else first.to(self.dtype)
        return linear(x0, self.w_first, None, out_dtype=torch.float32)

    def forward(self, residual, prepared, t):
        """The stream for pass t, written into `residual` (float32 [T, H])."""
        if not 0 <= t < self.passes:
            raise ValueError("pass %d of %d" % (t, self.passes))
        x = residual if self.dtype == torch.float32 else residual.to(self.dtype)
        y = linear(x, self.w_stream, None, out_dtype=torch.float32)
        torch.add(y, prepared, out=residual)
        residual.add_(self.steps[t])
        return residual
