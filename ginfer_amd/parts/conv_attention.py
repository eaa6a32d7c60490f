"""Attention whose projections pass a short convolution over time, with values of their own width and a sink."""
import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import Part, KVCacheSpec, StateSpec
from .linear import linear
from .registry import register_mixer


def _ceil16(n):
    return -(-int(n) // 16) * 16


@register_mixer("conv_attention")
class ConvAttention(Part):
    """q = Wq x, k = Wk x, v = Wv x (no biases); each channel of q, k and v then passes a causal convolution of `taps`
    taps over time (zeros before the sequence; the last taps - 1 projected rows of a request are its state); q and k are
    rotated by position (the rotary part may cover only the first coordinates of a head); grouped queries over the
    paged cache, scores times `scale`; `sink`: a score that every query sees beside its keys' and that has no value
    (None: a plain softmax); Wo on the heads' results.  Keys are head_dim wide, values value_dim.

    The attention kernels take one head size, so inside the part every head is `padded` = the wider of the two widths,
    rounded up to 16: the stacked projection matrix has rows of zeros where a head is narrower, the convolution's
    weights and Wo's columns likewise.  What the zeros add to a score or a result is exactly nothing."""

    capturable = True

    def __init__(self, hidden_size, num_heads, num_kv_heads, head_dim, value_dim, scale, dtype, device, taps=None,
                 position=None, sink=None, window=None, names=None):
        if num_heads % num_kv_heads:
            raise ValueError("num_heads %d is not a multiple of num_kv_heads %d" % (num_heads, num_kv_heads))
        self.hidden_size, self.nh, self.nkv = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.hd, self.vd = int(head_dim), int(value_dim)
        self.padded = _ceil16(max(self.hd, self.vd))
        if not 0 < self.padded <= 256:
            raise ValueError("heads of %d / %d are not supported: the attention kernels take head sizes up to 256"
                             % (self.hd, self.vd))
        self.taps = int(taps) if taps else 1
        if not 1 <= self.taps <= ops.SHORT_CONV_MAX_TAPS:
            raise ValueError("the short convolution takes 1 to %d taps, got %r" % (ops.SHORT_CONV_MAX_TAPS, taps))
        self.has_conv = bool(taps)
        self.position = position
        if position is not None and position.rotary_dim > self.hd:
            raise ValueError("the rotation covers %d coordinates of a head of %d" % (position.rotary_dim, self.hd))
        self.scale = float(scale)
        self.sink = None if sink is None else float(sink)
        self.window = int(window) if window else None
        self.names = dict(q="q", k="k", v="v", o="o", conv="conv")
        self.names.update(names or {})
        self.dtype, self.device = dtype, device
        self.width = (self.nh + 2 * self.nkv) * self.padded
        self.w_qkv = self.w_conv = self.w_o = self.sinks = self._no_rotation = None

    def cache_spec(self):
        """[the convolution's state (or None), the pages of keys and values]."""
        state = StateSpec((self.taps - 1, self.width), torch.float32) if self.taps > 1 else None
        return [state, KVCacheSpec(self.nkv, self.padded, self.window)]

    def weight_specs(self):
        n, H = self.names, self.hidden_size
        rows = {"q": self.nh * self.hd, "k": self.nkv * self.hd, "v": self.nkv * self.vd}
        specs = {n[r]: WeightSpec((rows[r], H)) for r in ("q", "k", "v")}
        specs[n["o"]] = WeightSpec((H, self.nh * self.vd))
        if self.has_conv:
            for r in ("q", "k", "v"):
                specs[n[r] + "." + n["conv"]] = WeightSpec((rows[r], self.taps), std=0.5, keep_32bit=True)
        return specs

    def _padded_rows(self, t, heads, width):
        """t [heads * width, ...] -> [heads * padded, ...] with zeros behind every head's rows."""
        if width == self.padded:
            return t
        out = torch.zeros((heads, self.padded) + tuple(t.shape[1:]), dtype=t.dtype, device=t.device)
        out[:, :width] = t.reshape((heads, width) + tuple(t.shape[1:]))
        return out.reshape((heads * self.padded,) + tuple(t.shape[1:]))

    def bind_weights(self, t):
        n = self.names
        heads = {"q": (self.nh, self.hd), "k": (self.nkv, self.hd), "v": (self.nkv, self.vd)}
        self.w_qkv = torch.cat([self._padded_rows(t[n[r]], *heads[r]) for r in ("q", "k", "v")], dim=0).contiguous()
        if self.has_conv:
            self.w_conv = torch.cat([self._padded_rows(t[n[r] + "." + n["conv"]].float(), *heads[r])
                                     for r in ("q", "k", "v")], dim=0).contiguous()
        w_o = t[n["o"]]
        self.w_o = self._padded_rows(w_o.t().contiguous(), self.nh, self.vd).t().contiguous()
        dev = self.w_qkv.device
        self.sinks = None if self.sink is None else torch.full((self.nh,), self.sink, dtype=torch.float32, device=dev)
        if self.position is None:                # the cache-writing kernel rotates by tables: angle zero everywhere
            self._no_rotation = (torch.ones((1, 1), dtype=torch.float32, device=dev),
                                 torch.zeros((1, 1), dtype=torch.float32, device=dev))

    def kernel_modules(self):
        mods = ["rope_kv", "attention_generic", "gemm", "short_conv"]
        if self.dtype == torch.bfloat16:
            mods += ["gemm_skinny"]
            if self.padded in ops.MFMA_HEAD_DIMS:
                mods += [("attention_mfma", {"HEAD_DIM": self.padded})]
        return mods

    def forward(self, x, step, cache):
        state, kv = cache
        if self.has_conv:
            # the convolution works on 32-bit rows and hands on the compute dtype
            proj = linear(x, self.w_qkv, None, out_dtype=torch.float32)
            if state is None:
                qkv = ops.short_conv(proj, self.w_conv, None, None, step, self.dtype, add_input=False)
            else:
                qkv = ops.short_conv(proj, self.w_conv, state.state, state.slots, step, self.dtype, add_input=False,
                                     update=state.owner)
        else:
            qkv = linear(x, self.w_qkv, None)
        if self.position is not None:
            cos, sin = self.position.tables()
            positions = step.positions
        else:
            cos, sin = self._no_rotation
            positions = torch.zeros_like(step.positions)
        ops.rope_kv_write(qkv, positions, cos, sin, kv.slot_mapping, kv.k_pages, kv.v_pages, self.nh, self.nkv,
                          self.padded, write_kv=kv.owner)
        a = ops.paged_attention(qkv, kv.k_pages, kv.v_pages, kv.block_table, step, self.nh, self.nkv, self.padded,
                                self.scale, self.window, sinks=self.sinks)
        return linear(a, self.w_o, None)
