"""A plain, slow implementation of the Videdra decoder: whole sequences, no cache, one function
per mechanism, float32 (or float64) tensors on the CPU.  It shares no code with the package:
it reads a model folder through the ``safetensors`` package and its own reading of
``config.json``.

The design, in this file's notation (x a token's row, W stored [out, in] and applied as W x):

* a layer:  s <- s + ls1 * n1b(mixer(n1(s)));  s <- s + ls2 * n2b(ff(n2(s)))  with four RMS
  norms n(x) = x / sqrt(mean(x^2) + eps) * w and two stored vectors ls1, ls2;
* mixer "attention": differential attention (two score maps per head over shared values) with
  grouped keys, a partly turned head, a window that keeps the first tokens, a per-head output
  gate, possibly reading another layer's keys and values;
* mixer "retention": a decayed outer-product state per head, read by the query;
* feed-forward: gated dense (tanh-gelu) or routed experts (silu) with a gated shared expert.
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


def rms_norm(x, weight, eps):
    """x / sqrt(mean(x^2) + eps) (* weight), over the last axis."""
    y = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def turn(x, positions, dims, base):
    """x [T, heads, d]: the first `dims` of every head turn, dim i with dim i + dims/2, by the
    angle position * base^(-2i/dims)."""
    if dims == 0:
        return x
    half = dims // 2
    i = torch.arange(half, dtype=torch.float64)
    freq = (float(base) ** (-2.0 * i / dims))
    angle = positions.to(torch.float64)[:, None] * freq[None, :]
    cos, sin = angle.cos().to(x.dtype)[:, None, :], angle.sin().to(x.dtype)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


def visible(n, size, keep_first):
    """[n, n] bool: query i sees key j."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    return (j <= i) & ((i - j < size) | (j < keep_first))


def _rot(m):
    rot = m.get("rot") or {}
    return rot.get("dims", 0), rot.get("base", 10000.0)


def attention_keys_values(h, w, prefix, m, positions, r=same):
    """The turned keys [T, G, 2, dim] and the values [T, G, vdim] a layer stores."""
    T = h.shape[0]
    G, dim, vdim = m["kv_heads"], m["dim"], m["vdim"]
    k = (h @ w[prefix + "k"].T).view(T, G * 2, dim)
    k = r(turn(k, positions, *_rot(m))).view(T, G, 2, dim)
    v = r(h @ w[prefix + "v"].T).view(T, G, vdim)
    return k, v


def differential_attention(h, w, prefix, m, eps, positions, kv=None, r=same):
    """h [T, width] -> [T, width].  `kv`: another layer's (keys, values) to read in place of
    this layer's own."""
    T = h.shape[0]
    H, G, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[prefix + "q"].T).view(T, H * 2, dim)
    q = r(turn(q, positions, *_rot(m))).view(T, H, 2, dim)
    k, v = kv if kv is not None else attention_keys_values(h, w, prefix, m, positions, r)
    mask_cfg = m.get("mask") or {}
    mask = visible(T, mask_cfg.get("size") or T + 1, mask_cfg.get("keep_first") or 0)
    lam = (torch.exp((w[prefix + "lq1"] * w[prefix + "lk1"]).sum())
           - torch.exp((w[prefix + "lq2"] * w[prefix + "lk2"]).sum()) + m["diff"])
    gate = torch.sigmoid(h @ w[prefix + "g"].T)                      # [T, H]
    out = torch.empty(T, H, vdim, dtype=h.dtype)
    per = H // G
    for head in range(H):
        g = head // per
        maps = []
        for which in range(2):
            score = (q[:, head, which] @ k[:, g, which].T) * m["scale"]
            score = score.masked_fill(~mask, float("-inf"))
            maps.append(r(torch.softmax(score, dim=-1) @ v[:, g]))
        o = maps[0] - lam * maps[1]
        o = rms_norm(o, None, eps) * (1.0 - m["diff"])
        out[:, head] = o * gate[:, head:head + 1]
    return r(out.reshape(T, H * vdim)) @ w[prefix + "o"].T


def retention(h, w, prefix, m, eps, positions, r=same, state=None):
    """`state` [H, dim, vdim] (default zeros) is where the recurrence starts; it is updated in
    place, so that a sequence can be run in pieces."""
    T = h.shape[0]
    H, dim, vdim = m["heads"], m["dim"], m["vdim"]
    q = turn((h @ w[prefix + "q"].T).view(T, H, dim), positions, *_rot(m))
    k = turn((h @ w[prefix + "k"].T).view(T, H, dim), positions, *_rot(m))
    k = k * dim ** -0.5
    v = (h @ w[prefix + "v"].T).view(T, H, vdim)
    out = torch.empty(T, H, vdim, dtype=h.dtype)
    for head in range(H):
        decay = float(m["decay"][head])
        s = torch.zeros(dim, vdim, dtype=h.dtype) if state is None else state[head]
        for t in range(T):
            s = decay * s + torch.outer(k[t, head], v[t, head])
            out[t, head] = s.T @ q[t, head]
        if state is not None:
            state[head] = s
    out = rms_norm(out, None, eps).reshape(T, H * vdim)
    return r(out * silu(h @ w[prefix + "g"].T)) @ w[prefix + "o"].T


def gated(h, w, prefix, act, r=same):
    return r(act(r(h @ w[prefix + "gate"].T)) * r(h @ w[prefix + "up"].T)) @ w[prefix + "down"].T


def routing_gap(logits, top):
    """[T]: how far the last chosen logit lies above the first one left out, relative to the
    largest logit's size (1 where every expert is chosen)."""
    if top >= logits.shape[-1]:
        return torch.ones(logits.shape[0], dtype=logits.dtype)
    ranked = logits.sort(-1, descending=True).values
    return (ranked[:, top - 1] - ranked[:, top]) / ranked.abs().amax(-1).clamp_min(1e-30)


def routed_experts(h, w, prefix, mlp, r=same, gaps=None):
    experts, top = mlp["router"]["experts"], mlp["router"]["top"]
    logits = h @ w[prefix + "router"].T
    if gaps is not None:
        gaps.append(routing_gap(logits, top))
    chosen, ids = torch.topk(logits, top, dim=-1)
    weights = torch.softmax(chosen, dim=-1)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(ids[t, j])
            out[t] += weights[t, j] * gated(h[t:t + 1], w, f"{prefix}e{e}.", silu, r)[0]
    if mlp.get("shared"):
        share = torch.sigmoid(h @ w[prefix + "shared.sg"].T)          # [T, 1]
        out = out + share * gated(h, w, prefix + "shared.", silu, r)
    return out


def feed_forward(h, w, prefix, mlp, r=same, gaps=None):
    if mlp["kind"] == "dense":
        return gated(h, w, prefix, gelu_tanh, r)
    return routed_experts(h, w, prefix, mlp, r, gaps)


def forward(config, w, tokens, r=same, return_layers=False, gaps=None):
    """Logits [T, vocab] of one sequence (and the stream after every layer).  `r` rounds what
    enters and leaves the matrix products (`to_bf16`: what the format costs on this input).
    `gaps`, a list, receives every routed layer's routing gaps [T]."""
    eps = config["norm"]["eps"]
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    positions = torch.arange(tokens.numel())
    s = w["embed"][tokens]
    stored, after = {}, []
    for i, layer in enumerate(config["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        h = r(rms_norm(s, w[p + "norm1"], eps))
        if layer["type"] == "attention":
            source = m.get("kv_from")
            if source is None:
                stored[i] = attention_keys_values(h, w, p + "mix.", m, positions, r)
            y = differential_attention(h, w, p + "mix.", m, eps, positions,
                                       kv=None if source is None else stored[source], r=r)
        elif layer["type"] == "retention":
            y = retention(h, w, p + "mix.", m, eps, positions, r)
        else:
            raise ValueError(layer["type"])
        s = s + w[p + "ls1"] * rms_norm(y, w[p + "norm1b"], eps)
        if layer.get("mlp"):
            h = r(rms_norm(s, w[p + "norm2"], eps))
            y = feed_forward(h, w, p + "mlp.", layer["mlp"], r, gaps)
            s = s + w[p + "ls2"] * rms_norm(y, w[p + "norm2b"], eps)
        after.append(s)
    logits = r(rms_norm(s, w["final.norm"], eps)) @ w["head"].T
    return (logits, torch.stack(after)) if return_layers else logits


def greedy_generate(config, w, prompt, count):
    """`count` tokens after `prompt`, each the largest logit of the whole sequence run anew."""
    tokens = list(prompt)
    for _ in range(count):
        tokens.append(int(forward(config, w, tokens)[-1].argmax()))
    return tokens[len(prompt):]
