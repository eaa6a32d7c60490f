"""A plain, slow statement of the Potupel decoder: whole sequences, no cache, one function per mechanism.

Written from the design's equations and sharing no code with the product package: model folders are read with the
`safetensors` package, every tensor stays on the CPU, and every call recomputes the whole sequence in float64.

The design, in this file's notation.  x is the residual stream [T, W]; x0 the embedding's output.
  embedding   x_t = E[id_t]
  norm_c      y = x / sqrt(mean(x^2) + eps) * (1 + g): the gain is stored around zero
  layer       x <- x + s1 * norm_c(mixer(norm_c(x)));  x <- x + s2 * norm_c(ff(norm_c(x)))   (ff may be absent);
              four norms with gains of their own, s1 and s2 one factor per channel
  loop        layers [start, stop) run `times` times with the same weights; before pass t:
              x <- Win [x; x0] + step[t]
  attention   q = Wq h, k = Wk h, v = Wv h; each goes through a causal convolution over time on every channel
              (c_t = sum_j w[:, j] * u_(t - taps + 1 + j), zeros before the sequence); q and k are rotated on their
              first `dims` coordinates (coordinate i pairs with i + dims/2, angle p * f_i); the frequencies f_i =
              base^(-2i/dims) are rescaled by wavelength; s_ij = scale * q_i . k_j for j <= i;
              p_ij = exp(s_ij) / (1 + sum_j exp(s_ij));  out = Wo concat_h sum_j p_ij v_j
  ff dense    Wdown relu(Wup h)^2
  ff routed   z = Wr h + b; the `top` largest z are chosen, weights = softmax over the chosen z;
              y = sum_e weight_e * expert_e(h) + shared(h);  expert(h) = Wdown (silu(Wgate h) * (Wup h))
  output      logits = E norm_c(x)
"""
import json
import math
import os

import torch

F64 = torch.float64


def read_config(folder):
    with open(os.path.join(folder, "config.json")) as f:
        return json.load(f)


def read_weights(folder, dtype=F64):
    from safetensors import safe_open
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            tensors[name] = f.get_tensor(name).to(dtype)
    return tensors


def centered_norm(x, g, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * (1.0 + g)


def channel_convolution(u, w):
    """u [T, C], w [C, taps]: c_t = sum_j w[:, j] * u_(t - taps + 1 + j)."""
    T, taps = u.shape[0], w.shape[1]
    out = torch.zeros_like(u)
    for j in range(taps):
        back = taps - 1 - j
        if back < T:
            out[back:] += w[:, j] * u[:T - back]
    return out


def rotary_frequencies(rot):
    """f_i for i < dims/2, rescaled by wavelength where the configuration says so.  32-bit, as the design computes."""
    dims = rot["dims"]
    out = []
    sc = rot.get("scaling")
    for i in range(dims // 2):
        f = float(rot["base"]) ** (-2.0 * i / dims)
        if sc:
            wavelength = 2.0 * math.pi / f
            if wavelength > sc["original"] / sc["low"]:
                f = f / sc["factor"]
            elif not wavelength < sc["original"] / sc["high"]:
                s = (sc["original"] / wavelength - sc["low"]) / (sc["high"] - sc["low"])
                f = (1.0 - s) * f / sc["factor"] + s * f
        out.append(f)
    return torch.tensor(out, dtype=F64).to(torch.float32)


def rotate(u, heads, dim, rot, first_position=0):
    """u [T, heads * dim]: the first rot.dims coordinates of every head turn by the position's angles."""
    T = u.shape[0]
    dims = rot["dims"]
    half = dims // 2
    pos = torch.arange(first_position, first_position + T, dtype=torch.float32)
    ang = (pos[:, None] * rotary_frequencies(rot)[None, :]).to(F64)       # the 32-bit product, as the design has it
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u = u.reshape(T, heads, dim).clone()
    a, b = u[..., :half].clone(), u[..., half:dims].clone()
    u[..., :half] = a * c - b * s
    u[..., half:dims] = b * c + a * s
    return u.reshape(T, heads * dim)


def sink_softmax_attention(q, k, v, heads, kv_heads, dim, vdim, scale, sink_scores=None):
    """q [T, heads*dim], k [T, kv_heads*dim], v [T, kv_heads*vdim] -> [T, heads*vdim]; causal, one added to the
    denominator of the softmax: a sink whose score is 0 (the design's; sink_scores gives every head another, for tests
    of the mechanism) and which has no value."""
    T = q.shape[0]
    q = q.reshape(T, heads, dim)
    k = k.reshape(T, kv_heads, dim)
    v = v.reshape(T, kv_heads, vdim)
    out = torch.zeros((T, heads, vdim), dtype=q.dtype)
    per = heads // kv_heads
    seen = torch.ones((T, T), dtype=torch.bool).tril()
    for h in range(heads):
        g = h // per
        s = ((q[:, h] @ k[:, g].T) * scale).masked_fill(~seen, -math.inf)
        sink = 0.0 if sink_scores is None else float(sink_scores[h])
        top = s.max(dim=-1, keepdim=True).values.clamp_min(sink)
        e = torch.exp(s - top)
        out[:, h] = (e / (torch.exp(sink - top) + e.sum(dim=-1, keepdim=True))) @ v[:, g]
    return out.reshape(T, heads * vdim)


def attention(h, w, p, m):
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q, k, v = h @ w[p + ".q"].T, h @ w[p + ".k"].T, h @ w[p + ".v"].T
    if m.get("conv"):
        q = channel_convolution(q, w[p + ".q.conv"])
        k = channel_convolution(k, w[p + ".k.conv"])
        v = channel_convolution(v, w[p + ".v.conv"])
    if m.get("rot"):
        q, k = rotate(q, H, D, m["rot"]), rotate(k, G, D, m["rot"])
    return sink_softmax_attention(q, k, v, H, G, D, V, m["scale"]) @ w[p + ".o"].T


def squared_relu_ff(h, w, p):
    return torch.relu(h @ w[p + ".up"].T) ** 2 @ w[p + ".down"].T


def gated_expert(h, w, p):
    g = h @ w[p + ".gate"].T
    return (g * torch.sigmoid(g) * (h @ w[p + ".up"].T)) @ w[p + ".down"].T


def route(h, w, p, experts, top):
    """Chosen experts [T, top] and their weights [T, top]."""
    z = h @ w[p + ".router"].T + w[p + ".router.b"]
    chosen = torch.topk(z, top, dim=-1)
    return chosen.indices, torch.softmax(chosen.values, dim=-1)


def routed_ff(h, w, p, mlp):
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    ids, weights = route(h, w, p, E, top)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(top):
            out[t] += weights[t, j] * gated_expert(h[t:t + 1], w, "%s.e%d" % (p, int(ids[t, j])))[0]
    if mlp.get("shared"):
        out = out + gated_expert(h, w, p + ".shared")
    return out


def feed_forward(h, w, p, mlp):
    return squared_relu_ff(h, w, p) if mlp["kind"] == "dense" else routed_ff(h, w, p, mlp)


def layer(x, w, i, l, eps):
    p = "l%d" % i
    m = attention(centered_norm(x, w[p + ".norm1"], eps), w, p + ".mix", l["mixer"])
    x = x + w[p + ".ls1"] * centered_norm(m, w[p + ".norm1b"], eps)
    if l.get("mlp"):
        f = feed_forward(centered_norm(x, w[p + ".norm2"], eps), w, p + ".mlp", l["mlp"])
        x = x + w[p + ".ls2"] * centered_norm(f, w[p + ".norm2b"], eps)
    return x


def layer_runs(cfg):
    """The order in which layers run: (layer, pass number if a pass starts before it else None)."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    runs = [(i, None) for i in range(loop["start"])]
    for t in range(loop["times"]):
        runs += [(i, t if i == loop["start"] else None) for i in range(loop["start"], loop["stop"])]
    return runs + [(i, None) for i in range(loop["stop"], n)]


def residual_streams(ids, w, cfg):
    """The stream after every layer run, [runs, T, W]."""
    eps = cfg["norm"]["eps"]
    x0 = w["embed"][torch.tensor(ids, dtype=torch.long)]
    x = x0
    out = []
    for i, t in layer_runs(cfg):
        if t is not None:
            x = torch.cat([x, x0], dim=-1) @ w["loop.in"].T + w["loop.step"][t]
        x = layer(x, w, i, cfg["layers"][i], eps)
        out.append(x)
    return torch.stack(out)


def logits(ids, w, cfg):
    x = residual_streams(ids, w, cfg)[-1]
    return centered_norm(x, w["final.norm"], cfg["norm"]["eps"]) @ w["embed"].T
