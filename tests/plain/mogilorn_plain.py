"""A plain, slow Mogilorn: whole sequences, no cache, one function per mechanism.

It shares no code with the package.  `weights` is a dict of tensors under the stored names
(``embed``, ``l<i>.norm1``, ``l<i>.mix.q``, ``l<i>.mix.q.b``, ``l<i>.mlp.up``, ``final.norm``),
`config` the model's configuration as a dict.  Everything is computed in `dtype` (float64 for
a reference, float32 for what 32-bit arithmetic costs); with `rounding` the operands of the
matrix products are rounded to bfloat16 first, which is what serving in bfloat16 costs.
"""

from __future__ import annotations

import math

import torch


def rounded(t: torch.Tensor, rounding: bool) -> torch.Tensor:
    return t.to(torch.bfloat16).to(t.dtype) if rounding else t


def linear(x, w, b=None, rounding=False):
    """W x (+ b) for a weight stored [out, in]."""
    y = rounded(x, rounding) @ w.to(x.dtype).T
    return y if b is None else y + b.to(x.dtype)


def rms(x, eps):
    """x over the root of (its mean square + eps), along the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def frequencies(rot: dict, dtype) -> torch.Tensor:
    """Angle per position step of every pair: base^(-2i/dims), and, with `scaling`, slowed
    where the wavelength is long (divided by `factor` beyond original/low, untouched below
    original/high, blended linearly in 1/wavelength between)."""
    dims = rot["dims"]
    f = torch.tensor([rot["base"] ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64)
    s = rot.get("scaling")
    if s:
        out = []
        for fi in f.tolist():
            wavelength = 2.0 * math.pi / fi
            if wavelength < s["original"] / s["high"]:
                out.append(fi)
            elif wavelength > s["original"] / s["low"]:
                out.append(fi / s["factor"])
            else:
                t = (s["original"] / wavelength - s["low"]) / (s["high"] - s["low"])
                out.append((1.0 - t) * fi / s["factor"] + t * fi)
        f = torch.tensor(out, dtype=torch.float64)
    return f.to(dtype)


def turn(x, positions, rot: dict):
    """Rotate the first rot['dims'] dims of the last axis, pairs (2i, 2i + 1), by
    position * frequency_i.  x: [T, heads, d]."""
    dims = rot["dims"]
    f = frequencies(rot, x.dtype)
    a = positions.to(x.dtype)[:, None] * f[None, :]            # [T, dims/2]
    cos, sin = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


def softmax_attention(q, k, v, scale, window=None, softcap=None, sink=None, rounding=False):
    """q [T, H, d], k [T, G, d], v [T, G, dv] of one sequence from its first token on; query
    head h reads key head h // (H / G).  Position i sees j <= i, with a window only
    i - j < window.  `softcap` bounds the scaled score through a tanh; `sink` [H] adds
    exp(sink_h) to the denominator."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[-1], dtype=q.dtype)
    i = torch.arange(T)
    seen = i[None, :] <= i[:, None]
    if window:
        seen &= (i[:, None] - i[None, :]) < window
    for h in range(H):
        g = h // (H // G)
        s = (rounded(q[:, h], rounding) @ rounded(k[:, g], rounding).T) * scale
        if softcap:
            s = softcap * torch.tanh(s / softcap)
        s = s.masked_fill(~seen, -math.inf)
        top = s.max(-1, keepdim=True).values
        if sink is not None:
            top = torch.maximum(top, sink[h].to(q.dtype).expand_as(top))
        e = torch.exp(s - top)
        denominator = e.sum(-1, keepdim=True)
        if sink is not None:
            denominator = denominator + torch.exp(sink[h].to(q.dtype) - top)
        out[:, h] = rounded(e / denominator, rounding) @ rounded(v[:, g], rounding)
    return out


def attention(h, positions, w, p, m, eps, v_first, rounding=False):
    """The 'attention' mixer.  Returns (output, this layer's unmixed values)."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = linear(h, w[p + "q"], w[p + "q.b"], rounding).view(T, H, d)
    k = linear(h, w[p + "k"], w[p + "k.b"], rounding).view(T, G, d)
    v = linear(h, w[p + "v"], w[p + "v.b"], rounding).view(T, G, dv)
    q = rms(q, eps) * w[p + "q.norm"].to(h.dtype)
    k = rms(k, eps) * w[p + "k.norm"].to(h.dtype)
    q, k = turn(q, positions, m["rot"]), turn(k, positions, m["rot"])
    own_v = v
    if m.get("v_mix") and v_first is not None:
        lam = w[p + "vmix"].to(h.dtype)
        v = (1.0 - lam) * v + lam * v_first
    o = softmax_attention(q, k, v, m["scale"], softcap=m.get("softcap"), rounding=rounding)
    gate = torch.sigmoid(linear(h, w[p + "g"], None, rounding))
    return linear(o.reshape(T, H * dv) * gate, w[p + "o"], w[p + "o.b"], rounding), own_v


def mlstm(h, w, p, m, eps, rounding=False, state=None):
    """The matrix-memory mixer, token by token.  `state` (S [H, d, dv], n [H, d], m [H]) is
    carried in and the new one returned beside the output."""
    T = h.shape[0]
    H, d, dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = linear(h, w[p + "q"], None, rounding).view(T, H, d) * d ** -0.5
    k = linear(h, w[p + "k"], None, rounding).view(T, H, d)
    v = linear(h, w[p + "v"], None, rounding).view(T, H, dv)
    i_gate = cap * torch.tanh(linear(h, w[p + "i"], w[p + "i.b"], rounding) / cap)          # [T, H]
    f_gate = torch.nn.functional.logsigmoid(
        cap * torch.tanh(linear(h, w[p + "f"], w[p + "f.b"], rounding) / cap))
    if state is None:
        S = torch.zeros(H, d, dv, dtype=h.dtype)
        n = torch.zeros(H, d, dtype=h.dtype)
        top = torch.zeros(H, dtype=h.dtype)
    else:
        S, n, top = (t.clone() for t in state)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for t in range(T):
        new_top = torch.maximum(f_gate[t] + top, i_gate[t])
        keep = torch.exp(f_gate[t] + top - new_top)
        take = torch.exp(i_gate[t] - new_top)
        S = keep[:, None, None] * S + take[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = keep[:, None] * n + take[:, None] * k[t]
        top = new_top
        above = torch.einsum("hdv,hd->hv", S, q[t])
        below = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-top)) + 1e-6
        out[t] = above / below[:, None]
    o = rms(out, eps).reshape(T, H * dv) * w[p + "norm"].to(h.dtype)
    o = o * torch.sigmoid(linear(h, w[p + "g"], None, rounding))
    return linear(o, w[p + "o"], None, rounding), (S, n, top)


def latent_attention(h, positions, w, p, m, eps, rounding=False):
    """The 'latent_attention' mixer: keys and values expanded from the normed latent."""
    T = h.shape[0]
    H, d, r, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = linear(h, w[p + "q"], None, rounding).view(T, H, d + r)
    down = linear(h, w[p + "dkv"], None, rounding)
    c = rms(down[:, :rank], eps) * w[p + "dkv.norm"].to(h.dtype)
    shared = down[:, rank:].view(T, 1, r)
    rot = dict(m["rot"], dims=r)
    q_turned = turn(q[..., d:], positions, rot)
    k_turned = turn(shared, positions, rot)
    k_plain = linear(c, w[p + "uk"], None, rounding).view(T, H, d)
    v = linear(c, w[p + "uv"], None, rounding).view(T, H, dv)
    q_all = torch.cat([q[..., :d], q_turned], -1)
    k_all = torch.cat([k_plain, k_turned.expand(T, H, r)], -1)
    window = (m.get("mask") or {}).get("size")
    o = softmax_attention(q_all, k_all, v, m["scale"], window=window, sink=w[p + "sink"],
                          rounding=rounding)
    gate = torch.sigmoid(linear(h, w[p + "g"], None, rounding))
    return linear(o.reshape(T, H * dv) * gate, w[p + "o"], None, rounding)


def feed_forward(h, w, p, rounding=False):
    return linear(gelu_tanh(linear(h, w[p + "up"], None, rounding)), w[p + "down"], None, rounding)


def norm_one_plus(x, weight, eps):
    return rms(x, eps) * (1.0 + weight.to(x.dtype))


def forward(config: dict, weights: dict, tokens, dtype=torch.float64, rounding=False,
            streams=None):
    """Logits [T, vocab] of one sequence from position 0.  `streams`, a list, receives the
    residual stream after every layer."""
    w = weights
    eps = config["norm"]["eps"]
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(len(tokens))
    x = w["embed"].to(dtype)[tokens] * config["embedding"]["scale"]
    v_first = None
    for i, layer in enumerate(config["layers"]):
        p, m = f"l{i}.mix.", layer["mixer"]
        if layer["type"] == "attention":
            y, own_v = attention(x, positions, w, p, m, eps, v_first, rounding)
            if m.get("v_mix") and v_first is None:
                v_first = own_v
        elif layer["type"] == "mlstm":
            y, _state = mlstm(x, w, p, m, eps, rounding)
        elif layer["type"] == "latent_attention":
            y = latent_attention(x, positions, w, p, m, eps, rounding)
        else:
            raise ValueError(layer["type"])
        x = x + norm_one_plus(y, w[f"l{i}.norm1"], eps)
        if layer.get("mlp"):
            x = x + norm_one_plus(feed_forward(x, w, f"l{i}.mlp.", rounding), w[f"l{i}.norm2"], eps)
        if streams is not None:
            streams.append(x.clone())
    x = norm_one_plus(x, w["final.norm"], eps)
    return linear(x, w["embed"], None, rounding)
