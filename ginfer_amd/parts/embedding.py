"""Token embedding and output head."""
import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import Part
from .linear import linear
from .registry import register_embedding, register_head


@register_embedding("embedding")
class Embedding(Part):
    """x[t, :] = E[ids[t], :], no scaling (ginfer/core/layer/embedding.cc:5-21); widened to the 32-bit
    residual stream as it is gathered."""

    capturable = True

    def __init__(self, vocab_size, hidden_size, dtype, device, weight_name="weight"):
        """weight_name: the table's name inside the part ("" where the checkpoint names it as the part itself)."""
        self.vocab_size, self.hidden_size, self.dtype, self.device = int(vocab_size), int(hidden_size), dtype, device
        self.weight_name = str(weight_name)
        self.weight = None

    def weight_specs(self):
        return {self.weight_name: WeightSpec((self.vocab_size, self.hidden_size))}

    def bind_weights(self, t):
        self.weight = t[self.weight_name]

    def kernel_modules(self):
        return ["embedding"]

    def forward(self, token_ids, step=None):
        return ops.embedding_gather(self.weight, token_ids)


@register_embedding("sinusoidal_normed")
class SinusoidalNormedEmbedding(Part):
    """x = norm(E[id] + P(p)): to the table's row a sinusoidal position vector is added, P[2i] = sin(p * base^(-2i/H)),
    P[2i+1] = cos of the same angle, and the sum goes through an RMS norm with one gain.  Angles are 32-bit: the
    position times a 32-bit frequency.  The table is named as the part itself, the gain `norm`."""

    capturable = True

    def __init__(self, vocab_size, hidden_size, eps, dtype, device, base=10000.0):
        self.vocab_size, self.hidden_size, self.eps, self.base = int(vocab_size), int(hidden_size), float(eps), float(base)
        self.dtype, self.device = dtype, device
        self.weight = self.gain = None
        i = torch.arange((self.hidden_size + 1) // 2, dtype=torch.float64)
        self._freq_host = torch.pow(torch.tensor(self.base, dtype=torch.float64), -2.0 * i / self.hidden_size).to(torch.float32)
        self._freq = None

    def weight_specs(self):
        return {"": WeightSpec((self.vocab_size, self.hidden_size), std=1.0),
                "norm": WeightSpec((), init="one_plus_normal", keep_32bit=True)}

    def bind_weights(self, t):
        self.weight = t[""]
        self.gain = t["norm"].float().reshape(1).contiguous()

    def kernel_modules(self):
        return ["embedding_sinusoid"]

    def forward(self, token_ids, step):
        if self._freq is None:
            self._freq = self._freq_host.to(self.weight.device)
        return ops.embedding_sinusoid_norm(self.weight, token_ids, step.positions, self._freq, self.gain, self.eps)


@register_head("lm_head")
class LMHead(Part):
    """logits = x . W^T, no bias, returned in 32-bit; W is the embedding table when tied
    (ginfer/core/layer/transformer/lmhead.cc:15-27, ginfer/model/qwen2.cc:42-46).  One device copy serves
    both uses when tied (the reference uploads it twice)."""

    capturable = True

    def __init__(self, vocab_size, hidden_size, tied, dtype, device, weight_name="weight"):
        """weight_name: the matrix's name inside the part ("" where the checkpoint names it as the part itself)."""
        self.vocab_size, self.hidden_size, self.tied = int(vocab_size), int(hidden_size), bool(tied)
        self.dtype, self.device = dtype, device
        self.weight_name = str(weight_name)
        self.weight = None

    def weight_specs(self):
        return {} if self.tied else {self.weight_name: WeightSpec((self.vocab_size, self.hidden_size))}

    def unread_weights(self):
        # a checkpoint of a tied model may still hold the head's copy of the table; like the reference
        # (ginfer/model/qwen2.cc:42-46) the model does not read it
        return [self.weight_name] if self.tied else []

    def bind_weights(self, t):
        if not self.tied:
            self.weight = t[self.weight_name]

    def tie(self, embedding_weight):
        self.weight = embedding_weight

    def kernel_modules(self):
        return ["gemm"] + (["gemm_skinny"] if self.dtype == torch.bfloat16 else [])

    def forward(self, x):
        return linear(x, self.weight, None, out_dtype=torch.float32)
