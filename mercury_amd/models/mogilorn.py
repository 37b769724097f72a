"""The Mogilorn decoder, put together from parts.

The embedding is multiplied by a stored-in-config scale.  A layer's sublayers read the float32
stream itself, and what they return is RMS-normed (weights stored around zero, 1 + w
multiplies) before it enters the stream: s += norm1(mixer(s)); s += norm2(ff(s)).  A layer of
type ``attention`` mixes with a grouped-query causal attention: biased projections, an RMS
norm per query and key head with one weight for all heads, interleaved rotation over a head's
first dims with frequencies slowed where the wavelength is long, a score bounded by a tanh,
values that (where the layer says so) are blended with the values the first such layer
projected for the same token, and a sigmoid gate per output column.  A layer of type
``mlstm`` carries a gated matrix memory per head and request.  A layer of type
``latent_attention`` attends through a normed latent and one rotated key part shared by the
heads, inside a sliding window, with a sink per head in the softmax's denominator and the
same kind of gate.  The feed-forward is down(gelu_tanh(up(x))), or absent.  The head is the
embedding, behind a final norm.
Tensors are stored without a ``.weight`` suffix and biases as ``.b``: ``embed``,
``l<i>.norm1``, ``l<i>.mix.q``, ``l<i>.mix.q.b``, ``l<i>.mix.q.norm``, ``l<i>.mix.vmix``,
``l<i>.mix.g``, ``l<i>.mix.i.b``, ``l<i>.mix.dkv.norm``, ``l<i>.mix.sink``, ``l<i>.mlp.up``,
``final.norm``.
"""

from __future__ import annotations

from ..config.model_config import MogilornConfig
from ..config.registry import register_architecture
from ..parts import (Attention, DecoderModel, LatentAttention, LayerCall, MatrixMemory, NoNorm,
                     NoPosition, PrePostNormBlock, RMSNorm, RotaryPosition, TokenEmbedding,
                     UnaryMLP)

BLOCK_NAMES = {"mixer": "mix.", "ffn": "mlp.", "norm_mixer": "unnormed1.", "norm_ffn": "unnormed2.",
               "post_mixer": "norm1.", "post_ffn": "norm2."}
ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm",
                   "gate": "g", "v_mix": "vmix"}
MEMORY_NAMES = {"q": "q", "k": "k", "v": "v", "gate": "g", "o": "o", "input": "i", "forget": "f",
                "norm": "norm"}
LATENT_NAMES = {"q": "q", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk", "uv": "uv", "o": "o",
                "sink": "sink", "gate": "g"}
FF_NAMES = {"up": "up", "down": "down"}


def stored_name(name: str) -> str:
    if name.endswith(".weight"):
        return name[:-len(".weight")]
    if name.endswith(".bias"):
        return name[:-len(".bias")] + ".b"
    return name


@register_architecture("Mogilorn", MogilornConfig)
def build_mogilorn(cfg: MogilornConfig) -> DecoderModel:
    positions: dict = {}    # one angle table per (width, base, turned dims, scaling)

    def position(width, base, dims, scaling):
        key = (width, base, dims, scaling)
        if key not in positions:
            positions[key] = (RotaryPosition(width, base, rotary_dim=dims, interleaved=True,
                                             scaling=scaling) if dims else NoPosition())
        return positions[key]

    post = lambda: RMSNorm(cfg.width, cfg.norm_eps, one_plus=True)
    mixing = cfg.mixing_layers()
    layers, calls = [], []
    for i, entry in enumerate(cfg.layers):
        m = entry.mixer
        if entry.kind == "attention":
            v_mix = None
            if m.v_mix and len(mixing) > 1:      # a lone such layer has nobody to mix with
                v_mix = "leave" if i == mixing[0] else "blend"
            mixer = Attention(
                cfg.width, m.heads, m.kv_heads, m.dim,
                position(m.dim, m.rot_base, m.rot_dims, m.rot_scaling), qkv_bias=True,
                o_bias=True, scale=m.scale, names=ATTENTION_NAMES, score_cap=m.softcap or None,
                value_dim=m.vdim, qk_norm="head", norm_eps=cfg.norm_eps, out_gate=True,
                v_mix=v_mix, v_mix_stored="yes" if m.v_mix else "maybe")
            calls.append(LayerCall(i, i))
        elif entry.kind == "mlstm":
            mixer = MatrixMemory(cfg.width, m.heads, m.dim, m.vdim, gate_cap=m.gate_cap or None,
                                 eps=cfg.norm_eps, names=MEMORY_NAMES)
            calls.append(LayerCall(i, None))
        else:
            mixer = LatentAttention(
                cfg.width, m.heads, m.dim, m.rot_dim, m.vdim, 0, m.kv_rank,
                position(m.rot_dim, m.rot_base, m.rot_dims, m.rot_scaling), cfg.norm_eps,
                scale=m.scale, window=m.window or None, names=LATENT_NAMES, sinks=True,
                out_gate=True)
            calls.append(LayerCall(i, i))
        ffn = UnaryMLP(cfg.width, entry.ff, "gelu_tanh", names=FF_NAMES) if entry.ff else None
        # (the norm behind a sublayer hands the new stream on in the compute dtype: only the
        # first layer copies it out by itself)
        layers.append(PrePostNormBlock(mixer, ffn, NoNorm(cfg.width), NoNorm(cfg.width) if ffn else None,
                                       post(), post() if ffn else None, BLOCK_NAMES,
                                       layer_scale=False, stream_given=i > 0,
                                       next_reads_stream=i + 1 < len(cfg.layers)))
    return DecoderModel(
        vocab_size=cfg.vocab, hidden_size=cfg.width, layers=layers,
        final_norm=RMSNorm(cfg.width, cfg.norm_eps, one_plus=True), tied_head=True, calls=calls,
        layer_prefix="l{}.", embed_name="embed.weight", norm_prefix="final.norm.",
        head_name="head.weight", max_positions=0, eos_token_ids=cfg.eos_token_ids, config=cfg,
        embedding=TokenEmbedding(cfg.vocab, cfg.width, scale=cfg.embedding_scale),
        stored_name=stored_name)
