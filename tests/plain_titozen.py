"""A plain, slow statement of the Titozen decoder: whole sequences, no cache, one function per mechanism.

Written from the design's equations and sharing no code with the product package: model folders are read
with the `safetensors` package, every tensor stays on the CPU, and every call recomputes the whole sequence.
The compute dtype is a parameter (float64 by default).

The design, in this file's notation.  x is the residual stream [T, W].
  embedding   x_t = norm_s(E[id_t] + P_t),   P_t[2i] = sin(t * 10000^(-2i/W)), P_t[2i+1] = cos(same)
  norm_s      y = g * x / sqrt(mean(x^2) + eps), g one number
  layer       h = x + conv(x);  x <- x + norm_s(mixer(h));  x <- x + norm_s(ff(x))   (ff may be absent)
  conv        conv(x)_t = sum_j w[:, j] * x_(t - taps + 1 + j), zeros before the sequence
  hgrn2       q = silu(Wq h), v = Wv h, f = l + (1 - l) * sigmoid(Wf h + b);  per head
              S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T,  o_t = S_t^T q_t;  out = Wo concat_h rms(o_t) * n
  latent attention   cq = rms(Wdq h) * nq, q = Wuq cq;  c = rms(Wdkv h) * nkv;  k = Wuk c, v = Wuv c per head;
              s_ij = scale * q_i . k_j for 0 <= i - j < window;  p_ij = exp(s_ij) / (exp(sink) + sum_j exp(s_ij));
              out = Wo concat_h (sigmoid(Wg h)_h * sum_j p_ij v_j)
  ff          g = min(Wgate x, L), u = clamp(Wup x, -L, L);  y = Wdown (g * sigmoid(1.702 g) * (u + 1))
  output      logits = Whead norm_s(x)
"""
import json
import math
import os

import torch


def read_config(folder):
    with open(os.path.join(folder, "config.json")) as f:
        return json.load(f)


def read_weights(folder, dtype=torch.float64):
    from safetensors import safe_open
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            tensors[name] = f.get_tensor(name).to(dtype)
    return tensors


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def scalar_norm(x, g, eps):
    return rms(x, eps) * g


def position_vectors(T, width, dtype):
    """Angles in 32-bit, as the design computes them: float(t) times a 32-bit frequency."""
    i = torch.arange((width + 1) // 2, dtype=torch.float64)
    freq = torch.pow(torch.tensor(10000.0, dtype=torch.float64), -2.0 * i / width).to(torch.float32)
    ang = torch.arange(T, dtype=torch.float32)[:, None] * freq[None, :]
    ang = ang.to(torch.float64)
    p = torch.zeros((T, width), dtype=torch.float64)
    p[:, 0::2] = torch.sin(ang)
    p[:, 1::2] = torch.cos(ang)[:, :width // 2]
    return p.to(dtype)


def embed(ids, w, cfg, dtype):
    x = w["embed"][torch.tensor(ids, dtype=torch.long)] + position_vectors(len(ids), cfg["width"], dtype)
    return scalar_norm(x, w["embed.norm"], cfg["norm"]["eps"])


def input_convolution(x, taps_w):
    """x [T, W], taps_w [W, taps]: x_t + sum_j w[:, j] * x_(t - taps + 1 + j)."""
    T, taps = x.shape[0], taps_w.shape[1]
    out = x.clone()
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += taps_w[:, j] * x[s]
    return out


def hgrn2(h, w, p, m, eps):
    """m: the mixer's sizes (heads, dim, vdim); p: prefix of its tensors."""
    H, D, V = m["heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = torch.nn.functional.silu(h @ w[p + "q"].T).view(T, H, D)
    v = (h @ w[p + "v"].T).view(T, H, V)
    lower = w[p + "lower"]
    f = (lower + (1 - lower) * torch.sigmoid(h @ w[p + "f"].T + w[p + "f.b"])).view(T, H, D)
    S = torch.zeros((H, D, V), dtype=h.dtype)
    out = torch.zeros((T, H, V), dtype=h.dtype)
    for t in range(T):
        S = f[t][:, :, None] * S + (1 - f[t])[:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    out = rms(out, eps) * w[p + "norm"]
    return out.reshape(T, H * V) @ w[p + "o"].T


def latent_attention(h, w, p, m, eps):
    H, D, V = m["heads"], m["dim"], m["vdim"]
    window, scale = m["mask"]["size"], m["scale"]
    T = h.shape[0]
    cq = rms(h @ w[p + "dq"].T, eps) * w[p + "dq.norm"]
    q = (cq @ w[p + "uq"].T).view(T, H, D)
    c = rms(h @ w[p + "dkv"].T, eps) * w[p + "dkv.norm"]
    k = (c @ w[p + "uk"].T).view(T, H, D)
    v = (c @ w[p + "uv"].T).view(T, H, V)
    gate = torch.sigmoid(h @ w[p + "g"].T)                 # [T, H]
    out = torch.zeros((T, H, V), dtype=h.dtype)
    for i in range(T):
        lo = max(0, i - window + 1)
        s = torch.einsum("hd,jhd->hj", q[i], k[lo:i + 1]) * scale           # [H, n]
        top = torch.maximum(s.max(dim=1).values, w[p + "sink"])
        e = torch.exp(s - top[:, None])
        den = e.sum(dim=1) + torch.exp(w[p + "sink"] - top)
        out[i] = torch.einsum("hj,jhv->hv", e / den[:, None], v[lo:i + 1]) * gate[i][:, None]
    return out.reshape(T, H * V) @ w[p + "o"].T


def feed_forward(x, w, p, mlp):
    if mlp["kind"] != "dense":
        raise ValueError("unknown feed-forward kind %r" % mlp["kind"])
    L = mlp["limit"]
    g = torch.clamp(x @ w[p + "gate"].T, max=L)
    u = torch.clamp(x @ w[p + "up"].T, -L, L)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ w[p + "down"].T


MIXERS = {"hgrn2": hgrn2, "latent_attention": latent_attention}


def forward(cfg, w, ids, dtype=torch.float64, layers_out=None):
    """Logits [T, vocab] for a whole sequence.  layers_out: a list that receives the residual stream after each layer."""
    eps = cfg["norm"]["eps"]
    x = embed(ids, w, cfg, dtype)
    for i, layer in enumerate(cfg["layers"]):
        p = "l%d." % i
        h = input_convolution(x, w[p + "canon1"])
        x = x + scalar_norm(MIXERS[layer["type"]](h, w, p + "mix.", layer["mixer"], eps), w[p + "norm1"], eps)
        if layer.get("mlp") is not None:
            x = x + scalar_norm(feed_forward(x, w, p + "mlp.", layer["mlp"]), w[p + "norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return scalar_norm(x, w["final.norm"], eps) @ w["head"].T


def logits(folder, ids, dtype=torch.float64):
    return forward(read_config(folder), read_weights(folder, dtype), ids, dtype).to(torch.float32).numpy()
