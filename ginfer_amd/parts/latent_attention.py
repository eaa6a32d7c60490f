"""Attention through a cached latent: queries and keys/values each pass a low-rank bottleneck, and only the latent of keys
and values is kept per token."""
import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import Part, PagedSpec
from .linear import linear
from .registry import register_mixer


@register_mixer("latent_attention")
class LatentAttention(Part):
    """cq = rms(Wdq h) * nq, q = Wuq cq;  c = rms(Wdkv h) * nkv, the latent (kv_rank numbers per token: all that is cached);
    per head k = Wuk c, v = Wuv c; scores scale * q . k over the last `window` positions (None: all), no position
    encoding; a softmax whose denominator also holds exp(sink) of a learned number per head (`sink=False`: none); each
    head's result times sigmoid(Wg h) of that head (`gated=False`: no gate); the heads side by side go through Wo.

    Since keys and values are linear in c, the attention runs in the latent space: qa = Wuk^T q per head, every head
    attends to the same cached rows c, as keys and as values, and Wuv is applied to the heads' results.  The three
    down-projections are one product, left in 32-bit for the norms and the gate; scores and softmax are 32-bit.
    Tensors: dq, dq.norm, uq, dkv, dkv.norm, uk, uv, sink, g, o."""

    capturable = True

    def __init__(self, hidden_size, num_heads, head_dim, value_dim, q_rank, kv_rank, scale, window, eps, dtype, device,
                 sink=True, gated=True):
        if not 0 < kv_rank <= ops.LATENT_MAX_RANK:
            raise ValueError("kv_rank %d is not supported: the latent attention kernel takes ranks up to %d"
                             % (kv_rank, ops.LATENT_MAX_RANK))
        self.hidden_size, self.nh, self.hd, self.vd = int(hidden_size), int(num_heads), int(head_dim), int(value_dim)
        self.q_rank, self.kv_rank = int(q_rank), int(kv_rank)
        self.scale = float(scale)
        self.window = int(window) if window else None
        self.eps, self.dtype, self.device = float(eps), dtype, device
        self.has_sink, self.gated = bool(sink), bool(gated)
        self.w_down = self.q_norm = self.kv_norm = self.w_uq = self.w_uk_t = self.w_uv = self.sink = self.w_o = None

    def cache_spec(self):
        """The latent per token, in pages.  Where the matrix-core kernel can run (bfloat16, a rank in steps of 8) a page holds
        a second copy, transposed ([rank][slot]): that kernel reads the latent as keys from the first and as values from
        the second, each in 16-byte operands."""
        if self.dtype == torch.bfloat16 and self.kv_rank % 8 == 0:
            return PagedSpec((("c", self.kv_rank), ("ct", self.kv_rank)), self.window)
        return PagedSpec((("c", self.kv_rank),), self.window)

    def weight_specs(self):
        H, nh = self.hidden_size, self.nh
        specs = {"dq": WeightSpec((self.q_rank, H)), "dq.norm": WeightSpec((self.q_rank,), init="one_plus_normal"),
                 "uq": WeightSpec((nh * self.hd, self.q_rank)), "dkv": WeightSpec((self.kv_rank, H)),
                 "dkv.norm": WeightSpec((self.kv_rank,), init="one_plus_normal"),
                 "uk": WeightSpec((nh * self.hd, self.kv_rank)), "uv": WeightSpec((nh * self.vd, self.kv_rank)),
                 "o": WeightSpec((H, nh * self.vd))}
        if self.has_sink:
            specs["sink"] = WeightSpec((nh,), std=0.2)
        if self.gated:
            specs["g"] = WeightSpec((nh, H))
        return specs

    def bind_weights(self, t):
        down = [t["dq"], t["dkv"]] + ([t["g"]] if self.gated else [])
        self.w_down = torch.cat(down, dim=0).contiguous()
        self.q_norm = t["dq.norm"].float().contiguous()
        self.kv_norm = t["dkv.norm"].float().contiguous()
        self.w_uq = t["uq"]
        self.w_uk_t = t["uk"].view(self.nh, self.hd, self.kv_rank).transpose(1, 2).contiguous()   # [head][rank][dim]
        self.w_uv = t["uv"].view(self.nh, self.vd, self.kv_rank).contiguous()                     # [head][vdim][rank]
        self.sink = t["sink"].float().contiguous() if self.has_sink else None
        self.w_o = t["o"]

    def kernel_modules(self):
        return ["latent_attention", "gemm"] + (["gemm_skinny"] if self.dtype == torch.bfloat16 else [])

    def forward(self, x, step, cache):
        T = x.shape[0]
        proj = linear(x, self.w_down, None, out_dtype=torch.float32)
        c_pages, ct_pages = cache.pages["c"], cache.pages.get("ct")
        cq, gate = ops.latent_prepare(proj, self.q_norm, self.kv_norm, cache.slot_mapping, c_pages, self.q_rank,
                                      self.kv_rank, self.nh, self.eps, self.dtype, write=cache.owner, gated=self.gated,
                                      ct_pages=ct_pages)
        q = linear(cq, self.w_uq).view(T, self.nh, self.hd).transpose(0, 1)                       # [head][T][dim]
        # the queries carried into the latent space, head by head, in 32-bit.  bfloat16: one batched product of the
        # library; float32: the package's own product per head, whose bits do not depend on the number of rows
        if self.dtype == torch.float32:
            qa = torch.empty((self.nh, T, self.kv_rank), dtype=torch.float32, device=x.device)
            for h in range(self.nh):
                ops.gemm_nt(q[h], self.w_uk_t[h], out=qa[h])
        else:
            qa = torch.bmm(q, self.w_uk_t.transpose(1, 2), out_dtype=torch.float32)
        a = ops.latent_attention(qa, c_pages, cache.block_table, step, self.sink, gate, self.nh, self.kv_rank,
                                 cache.page_size, self.scale, self.window, self.dtype, ct_pages=ct_pages)   # [head][T][rank]
        o = torch.empty((T, self.nh, self.vd), dtype=self.dtype, device=x.device)
        if self.dtype == torch.float32:
            for h in range(self.nh):
                ops.gemm_nt(a[h], self.w_uv[h], out=o[:, h])
        else:
            torch.bmm(a, self.w_uv.transpose(1, 2), out=o.transpose(0, 1))
        return linear(o.view(T, self.nh * self.vd), self.w_o)
