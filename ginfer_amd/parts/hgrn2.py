"""HGRN2: linear attention in which the forget gate also decides what is written, as a recurrence over per-request state."""
import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import Part, StateSpec
from .linear import linear
from .registry import register_mixer


@register_mixer("hgrn2")
class HGRN2(Part):
    """q = silu(Wq h), v = Wv h, f = l + (1 - l) * sigmoid(Wf h + b) with a lower bound l per head and channel; per head
    S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T and o_t = S_t^T q_t (no key of its own, no other scale); each head's o is
    RMS-normed over its value columns with a weight shared by the heads; the heads side by side go through Wo.
    The three projections are one product over the stacked weights, left in 32-bit; gates, state (32-bit, one slot per
    request, zeros at a request's start) and the output sum are 32-bit.  Tensors: q, f, f.b, lower, v, norm, o."""

    capturable = True

    def __init__(self, hidden_size, num_heads, key_dim, value_dim, eps, dtype, device):
        if not 0 < key_dim <= ops.HGRN2_MAX_DIM:
            raise ValueError("key_dim %d is not supported: the recurrence kernel takes up to %d channels per head"
                             % (key_dim, ops.HGRN2_MAX_DIM))
        self.hidden_size, self.nh, self.dk, self.dv = int(hidden_size), int(num_heads), int(key_dim), int(value_dim)
        self.eps, self.dtype, self.device = float(eps), dtype, device
        self.w_qfv = self.f_bias = self.lower = self.norm_weight = self.w_o = None

    def cache_spec(self):
        return StateSpec((self.nh, self.dk, self.dv), torch.float32)

    def weight_specs(self):
        H, k, v = self.hidden_size, self.nh * self.dk, self.nh * self.dv
        return {"q": WeightSpec((k, H)), "f": WeightSpec((k, H)), "f.b": WeightSpec((k,), std=0.2),
                "lower": WeightSpec((k,), init="unit_interval"), "v": WeightSpec((v, H)),
                "norm": WeightSpec((self.dv,), init="one_plus_normal"), "o": WeightSpec((H, v))}

    def bind_weights(self, t):
        self.w_qfv = torch.cat([t["q"], t["f"], t["v"]], dim=0).contiguous()
        self.f_bias = t["f.b"].float().contiguous()
        self.lower = t["lower"].float().contiguous()
        self.norm_weight = t["norm"].float().contiguous()
        self.w_o = t["o"]

    def kernel_modules(self):
        return ["gated_recurrence", "gemm"] + (["gemm_skinny"] if self.dtype == torch.bfloat16 else [])

    def forward(self, x, step, cache):
        proj = linear(x, self.w_qfv, None, out_dtype=torch.float32)
        o = ops.hgrn2_scan(proj, self.f_bias, self.lower, cache.state, cache.slots, step, self.nh, self.dk, self.dv,
                           update=cache.owner)
        o = ops.headwise_rmsnorm(o, self.norm_weight, self.eps, self.dtype)
        return linear(o.view(x.shape[0], self.nh * self.dv), self.w_o)
