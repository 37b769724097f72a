"""A plain, slow implementation of the Mogilorn decoder: whole sequences, no cache, one function
per mechanism, float32 (or float64) tensors on the CPU.  It shares no code with the package:
it reads a model folder through the ``safetensors`` package and its own reading of
``config.json``.

The design, in this file's notation (x a token's row, W stored [out, in] and applied as W x,
rms(x) = x / sqrt(mean(x^2) + eps)):

* the embedding row times ``embedding.scale`` starts the stream s;
* a layer:  s <- s + rms(mixer(s)) (1 + w1);  s <- s + rms(ff(s)) (1 + w2): the sublayers read
  s itself, their outputs are normed;
* mixer "attention": grouped keys and values, biased projections, rms per query and key head
  times one weight for all heads, pairs (2i, 2i + 1) of a head's first dims turned by
  position * frequency_i (frequencies slowed where the wavelength is long), the scaled score
  bounded by cap * tanh(. / cap), causal softmax, values blended with the first mixing layer's,
  the heads' outputs times sigmoid(W_g s), an output projection with a bias;
* mixer "mlstm": a gated outer-product memory per head with a running maximum;
* mixer "latent_attention": keys and values expanded from one normed latent a token plus one
  turned key part all heads share, a sliding window, a sink in the softmax's denominator, the
  same kind of gate;
* feed-forward: down(gelu_tanh(up(s))); the head is the embedding matrix behind a final norm.

`r` rounds what enters a matrix product (identity, or a round trip through bfloat16).
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch


def load_folder(folder, dtype=torch.float32):
    from safetensors import safe_open

    folder = Path(folder)
    config = json.loads((folder / "config.json").read_text())
    tensors = {}
    with safe_open(str(folder / "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            t = f.get_tensor(name)
            tensors[name] = t.to(dtype) if t.is_floating_point() else t
    return config, tensors


def to_bf16(t):
    """What a tensor is after a round trip through bfloat16."""
    return t.to(torch.bfloat16).to(t.dtype)


def same(t):
    return t


def read_config(folder) -> dict:
    return json.loads((Path(folder) / "config.json").read_text())


def read_weights(folder, dtype=torch.float32) -> dict:
    return load_folder(folder, dtype)[1]


def linear(x, w, b=None, r=same):
    y = r(x) @ w.T
    return y if b is None else y + b


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def frequencies(rot: dict) -> list:
    """Angle per position step of every pair.  With `scaling`: a wavelength below
    original / high keeps its frequency, one above original / low turns `factor` times slower,
    and between the two the slowed and the plain frequency are blended by
    t = (original / wavelength - low) / (high - low)."""
    dims, out = rot["dims"], []
    s = rot.get("scaling")
    for i in range(dims // 2):
        f = rot["base"] ** (-2.0 * i / dims)
        if s:
            wavelength = 2.0 * math.pi / f
            if wavelength > s["original"] / s["low"]:
                f = f / s["factor"]
            elif wavelength >= s["original"] / s["high"]:
                t = (s["original"] / wavelength - s["low"]) / (s["high"] - s["low"])
                f = (1.0 - t) * f / s["factor"] + t * f
        out.append(f)
    return out


def turn(x, positions, rot):
    """x [T, heads, d]: pairs (2i, 2i + 1) of the first rot['dims'] dims turned by the token's
    position times the pair's frequency; the other dims pass."""
    if not rot or not rot.get("dims"):
        return x
    dims = rot["dims"]
    f = torch.tensor(frequencies(rot), dtype=torch.float64)
    angle = (positions.to(torch.float64)[:, None] * f[None, :]).to(x.dtype)
    cos, sin = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


def visible(positions, window):
    """[T, T] bool: query i sees key j when j <= i and, with a window, i - j < window."""
    i, j = positions[:, None], positions[None, :]
    seen = j <= i
    if window:
        seen = seen & (i - j < window)
    return seen


def softmax_attention(q, k, v, positions, scale, window=0, softcap=0.0, sink=None, r=same):
    """q [T, H, d], k [T, G, d], v [T, G, dv]; query head h reads key head h // (H / G).
    `softcap` bounds the scaled score; `sink` [H]: exp(sink_h) once more in the denominator."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[-1], dtype=q.dtype)
    seen = visible(positions, window)
    for h in range(H):
        g = h // (H // G)
        s = (r(q[:, h]) @ r(k[:, g]).T) * scale
        if softcap:
            s = softcap * torch.tanh(s / softcap)
        s = s.masked_fill(~seen, -math.inf)
        top = s.max(-1, keepdim=True).values
        if sink is not None:
            top = torch.maximum(top, sink[h].expand_as(top))
        e = torch.exp(s - top)
        below = e.sum(-1, keepdim=True)
        if sink is not None:
            below = below + torch.exp(sink[h] - top)
        out[:, h] = r(e / below) @ r(v[:, g])
    return out


def attention_values(h, w, p, m, r=same):
    """The layer's own values as projected, [T, G, dv]."""
    return linear(h, w[p + "v"], w[p + "v.b"], r).view(h.shape[0], m["kv_heads"], m["vdim"])


def attention(h, w, p, m, eps, positions, v_first=None, r=same):
    """The 'attention' mixer; `v_first`, when given, is blended into the layer's values."""
    T, H, G, d, dv = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = linear(h, w[p + "q"], w[p + "q.b"], r).view(T, H, d)
    k = linear(h, w[p + "k"], w[p + "k.b"], r).view(T, G, d)
    v = attention_values(h, w, p, m, r)
    q = turn(rms(q, eps) * w[p + "q.norm"], positions, m.get("rot"))
    k = turn(rms(k, eps) * w[p + "k.norm"], positions, m.get("rot"))
    if v_first is not None:
        lam = w[p + "vmix"]
        v = (1.0 - lam) * v + lam * v_first
    o = softmax_attention(q, k, v, positions, m["scale"], softcap=m.get("softcap") or 0.0, r=r)
    gate = torch.sigmoid(linear(h, w[p + "g"], None, r))
    return linear(o.reshape(T, H * dv) * gate, w[p + "o"], w[p + "o.b"], r)


def matrix_memory(h, w, p, m, eps, r=same, state=None, return_state=False):
    """The 'mlstm' mixer, token by token; `state` = (S [H, d, dv], n [H, d], m [H])."""
    T, H, d, dv = h.shape[0], m["heads"], m["dim"], m["vdim"]
    cap = m.get("gate_cap") or 0.0
    q = linear(h, w[p + "q"], None, r).view(T, H, d) * d ** -0.5
    k = linear(h, w[p + "k"], None, r).view(T, H, d)
    v = linear(h, w[p + "v"], None, r).view(T, H, dv)
    a = linear(h, w[p + "i"], w[p + "i.b"], r)
    b = linear(h, w[p + "f"], w[p + "f.b"], r)
    if cap:
        a, b = cap * torch.tanh(a / cap), cap * torch.tanh(b / cap)
    log_in, log_keep = a, torch.nn.functional.logsigmoid(b)
    if state is None:
        S, n, top = h.new_zeros(H, d, dv), h.new_zeros(H, d), h.new_zeros(H)
    else:
        S, n, top = (t.clone() for t in state)
    out = h.new_zeros(T, H, dv)
    for t in range(T):
        new_top = torch.maximum(log_keep[t] + top, log_in[t])
        keep = torch.exp(log_keep[t] + top - new_top)
        take = torch.exp(log_in[t] - new_top)
        S = keep[:, None, None] * S + take[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = keep[:, None] * n + take[:, None] * k[t]
        top = new_top
        above = torch.einsum("hdv,hd->hv", S, q[t])
        below = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-top)) + 1e-6
        out[t] = above / below[:, None]
    o = rms(out, eps).reshape(T, H * dv) * w[p + "norm"]
    o = o * torch.sigmoid(linear(h, w[p + "g"], None, r))
    y = linear(o, w[p + "o"], None, r)
    return (y, (S, n, top)) if return_state else y


def latent_attention(h, w, p, m, eps, positions, r=same):
    """The 'latent_attention' mixer with every head's keys and values written out."""
    T, H, d, rd, dv, rank = h.shape[0], m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = linear(h, w[p + "q"], None, r).view(T, H, d + rd)
    down = linear(h, w[p + "dkv"], None, r)
    c = rms(down[:, :rank], eps) * w[p + "dkv.norm"]
    # the turned part turns whole unless the entry says how many of its dims do; no entry: none
    rot = dict(m["rot"], dims=m["rot"].get("dims", rd)) if rd and m.get("rot") else None
    q_turned = turn(q[..., d:], positions, rot)
    k_turned = turn(down[:, rank:].reshape(T, 1, rd), positions, rot)
    k_plain = linear(c, w[p + "uk"], None, r).view(T, H, d)
    v = linear(c, w[p + "uv"], None, r).view(T, H, dv)
    q_all = torch.cat([q[..., :d], q_turned], -1)
    k_all = torch.cat([k_plain, k_turned.expand(T, H, rd)], -1)
    window = (m.get("mask") or {}).get("size") or 0
    o = softmax_attention(q_all, k_all, v, positions, m["scale"], window=window, sink=w[p + "sink"], r=r)
    gate = torch.sigmoid(linear(h, w[p + "g"], None, r))
    return linear(o.reshape(T, H * dv) * gate, w[p + "o"], None, r)


def feed_forward(h, w, p, r=same):
    return linear(gelu_tanh(linear(h, w[p + "up"], None, r)), w[p + "down"], None, r)


def normed(y, weight, eps):
    """A sublayer's output before it enters the stream: the stored weight lies around zero."""
    return rms(y, eps) * (1.0 + weight)


def forward(config, w, tokens, r=same, return_layers=False):
    """Logits [T, vocab] of one sequence from position 0, in the dtype of the weights."""
    eps = config["norm"]["eps"]
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(len(tokens))
    s = w["embed"][tokens] * (config.get("embedding") or {}).get("scale", 1.0)
    mixing = [i for i, layer in enumerate(config["layers"])
              if layer["type"] == "attention" and layer["mixer"].get("v_mix")]
    v_first, layers = None, []
    for i, layer in enumerate(config["layers"]):
        p, m = f"l{i}.mix.", layer["mixer"]
        if layer["type"] == "attention":
            if mixing and i == mixing[0]:
                v_first = attention_values(s, w, p, m, r)
                y = attention(s, w, p, m, eps, positions, None, r)
            else:
                y = attention(s, w, p, m, eps, positions, v_first if i in mixing else None, r)
        elif layer["type"] == "mlstm":
            y = matrix_memory(s, w, p, m, eps, r)
        elif layer["type"] == "latent_attention":
            y = latent_attention(s, w, p, m, eps, positions, r)
        else:
            raise ValueError(layer["type"])
        s = s + normed(y, w[f"l{i}.norm1"], eps)
        if layer.get("mlp"):
            s = s + normed(feed_forward(s, w, f"l{i}.mlp.", r), w[f"l{i}.norm2"], eps)
        layers.append(s)
    logits = linear(normed(s, w["final.norm"], eps), w["embed"], None, r)
    return (logits, layers) if return_layers else logits


def greedy_generate(config, w, prompt, count):
    tokens = list(prompt)
    for _ in range(count):
        tokens.append(int(forward(config, w, tokens)[-1].argmax()))
    return tokens[len(prompt):]
