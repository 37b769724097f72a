"""The Videdra decoder, put together from parts.

Every layer norms before and after each sublayer and multiplies what enters the float32 stream
by a stored vector: s += ls1 * norm1b(mixer(norm1(s))); s += ls2 * norm2b(ff(norm2(s))).  A
layer of type ``attention`` mixes with a differential attention: two score maps a head (side
by side in the q and k projections, each turned over its first dims), both softmaxed over the
same grouped values inside a window that keeps the sequence's first tokens, combined as
a1 - lam * a2, normed per head, gated per head by a sigmoid of the mixer's input; with
``kv_from`` it reads an earlier layer's keys and values with queries, mask and everything else
of its own.  A layer of type ``retention`` carries a decayed outer-product state per head and
request.  The feed-forward is a tanh-gelu gated one, or routed SiLU experts (softmax over the
chosen logits) beside a shared expert gated by one sigmoid a token, or absent.
Tensors are stored without a ``.weight`` suffix: ``embed``, ``l<i>.norm1``, ``l<i>.norm1b``,
``l<i>.ls1``, ``l<i>.mix.q``, ``l<i>.mix.lq1``, ``l<i>.mix.g``, ``l<i>.mlp.e<k>.gate``,
``l<i>.mlp.router``, ``l<i>.mlp.shared.sg``, ``final.norm``, ``head``.
"""

from __future__ import annotations

from ..config.model_config import VidedraConfig
from ..config.registry import register_architecture
from ..parts import (Attention, DecoderModel, GatedMLP, LayerCall, NoPosition, PrePostNormBlock,
                     Retention, RMSNorm, RotaryPosition, RoutedExperts)

BLOCK_NAMES = {"mixer": "mix.", "ffn": "mlp.", "norm_mixer": "norm1.", "norm_ffn": "norm2.",
               "post_mixer": "norm1b.", "post_ffn": "norm2b.", "scale_mixer": "ls1",
               "scale_ffn": "ls2"}
ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "gate": "g", "lq1": "lq1", "lk1": "lk1",
                   "lq2": "lq2", "lk2": "lk2"}
RETENTION_NAMES = {"q": "q", "k": "k", "v": "v", "gate": "g", "o": "o"}
FF_NAMES = {"gate": "gate", "up": "up", "down": "down"}
# the design's constant: a head's two maps
MAPS = 2


def stored_name(name: str) -> str:
    return name[:-len(".weight")] if name.endswith(".weight") else name


def _feed_forward(cfg: VidedraConfig, mlp):
    if mlp is None:
        return None
    if mlp.kind == "dense":
        return GatedMLP(cfg.width, mlp.ff, "gelu_tanh", names=FF_NAMES)
    shared = GatedMLP(cfg.width, mlp.shared_ff, "silu", names=FF_NAMES) if mlp.shared_ff else None
    # the softmax over the chosen logits alone is the softmax over all, renormalised
    return RoutedExperts(cfg.width, mlp.experts, mlp.top, mlp.ff, scale=1.0, renormalize=True,
                         activation="silu", shared=shared, shared_gated=shared is not None)


def _cache_needs(cfg: VidedraConfig) -> dict:
    """Writing layer -> (window or None, kept first tokens) its cache slot must hold: the widest
    mask among the layer itself and the layers that read its keys and values."""
    needs: dict = {}
    for i, layer in enumerate(cfg.layers):
        if layer.kind != "attention":
            continue
        m = layer.mixer
        slot = i if m.kv_from is None else m.kv_from
        window, keep = needs.get(slot, (m.window, m.keep_first))
        if not window or not m.window:
            needs[slot] = (0, 0)
        else:
            needs[slot] = (max(window, m.window), max(keep, m.keep_first))
    return needs


@register_architecture("Videdra", VidedraConfig)
def build_videdra(cfg: VidedraConfig) -> DecoderModel:
    positions: dict = {}    # one angle table per (width, base, turned dims)

    def position(dim, base, dims):
        key = (dim, base, dims)
        if key not in positions:
            positions[key] = RotaryPosition(dim, base, rotary_dim=dims) if dims else NoPosition()
        return positions[key]

    # x * rstd * weight in float32, rounded once where a matrix product reads it
    norm = lambda: RMSNorm(cfg.width, cfg.norm_eps, round_once=True)
    needs = _cache_needs(cfg)
    layers, calls = [], []
    for i, entry in enumerate(cfg.layers):
        m = entry.mixer
        if entry.kind == "attention":
            own = m.kv_from is None
            window, keep = needs[i] if own else (m.window, m.keep_first)
            mixer = Attention(
                cfg.width, m.heads, m.kv_heads, MAPS * m.dim, position(m.dim, m.rot_base, m.rot_dims),
                qkv_bias=False, o_bias=False, scale=m.scale, window=m.window or None,
                names=ATTENTION_NAMES, value_dim=m.vdim, norm_eps=cfg.norm_eps,
                keep_first=m.keep_first, maps=MAPS, diff_init=m.diff, head_gate=True,
                cache_window=window or None, cache_keep_first=keep, own_kv=own)
            calls.append(LayerCall(i, i if own else m.kv_from, writes=own))
        else:
            mixer = Retention(cfg.width, m.heads, m.dim, m.vdim, m.decay,
                              position(m.dim, m.rot_base, m.rot_dims), eps=cfg.norm_eps,
                              names=RETENTION_NAMES)
            calls.append(LayerCall(i, None))
        ffn = _feed_forward(cfg, entry.mlp)
        layers.append(PrePostNormBlock(mixer, ffn, norm(), norm() if ffn else None, norm(),
                                       norm() if ffn else None, BLOCK_NAMES))
    return DecoderModel(
        vocab_size=cfg.vocab, hidden_size=cfg.width, layers=layers, final_norm=norm(),
        tied_head=False, calls=calls, layer_prefix="l{}.", embed_name="embed.weight",
        norm_prefix="final.norm.", head_name="head.weight", max_positions=0,
        eos_token_ids=cfg.eos_token_ids, config=cfg, stored_name=stored_name)
