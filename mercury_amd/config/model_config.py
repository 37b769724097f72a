"""Typed model configurations, read from an architecture's own ``config.json`` keys.

One dataclass per architecture; the registry in :mod:`mercury_amd.config.registry` maps the
``architectures[0]`` string of ``config.json`` to the dataclass and to the function that turns
it into a model description.  No size or constant that ``config.json`` gives is repeated in
code; the only defaults are the ones the reference applies when a key is absent
(reference: mercury/config.py:45-71).
"""

from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path


class ConfigError(ValueError):
    """config.json names something this engine does not implement, or lacks a key."""


def read_config_json(folder) -> dict:
    """The parsed ``config.json`` of a model folder (or the file itself, when given that)."""
    path = Path(folder)
    if path.is_dir() or path.name != "config.json":
        path = path / "config.json"
    if not path.is_file():
        raise FileNotFoundError(f"no config.json under {folder}")
    return json.loads(path.read_text())


def _require(raw: dict, key: str):
    if key not in raw:
        raise ConfigError(f"config.json has no {key!r}")
    return raw[key]


@dataclass(frozen=True)
class Qwen2Config:
    """The Qwen2 dense decoder (reference: mercury/config.py:22-71, mercury/model/qwen2.py).

    Keys and defaults follow the reference: ``num_key_value_heads`` defaults to the number of
    heads, ``head_dim`` to ``hidden_size // num_attention_heads``, ``rms_norm_eps`` to 1e-6,
    ``rope_theta`` to 10000, ``max_position_embeddings`` to 32768, ``tie_word_embeddings`` to
    false; ``eos_token_id`` may be an integer or a list.

    The reference never reads the sliding-window keys or ``rope_scaling`` or ``hidden_act``:
    its attention is always full and causal, its rotation unscaled and its activation SiLU
    (mercury/model/qwen2.py:42, mercury/model/attention.py:77-101).  A config that asks for
    anything else is refused here instead of being run with the wrong arithmetic.
    """

    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    vocab_size: int
    rms_norm_eps: float
    rope_theta: float
    max_position_embeddings: int
    tie_word_embeddings: bool
    eos_token_ids: tuple = ()
    bos_token_id: int | None = None
    architecture: str = "Qwen2ForCausalLM"

    @classmethod
    def from_dict(cls, raw: dict) -> "Qwen2Config":
        arch = (raw.get("architectures") or ["Qwen2ForCausalLM"])[0]
        heads = int(_require(raw, "num_attention_heads"))
        hidden = int(_require(raw, "hidden_size"))
        eos = raw.get("eos_token_id", [])
        if eos is None:
            eos = []
        if isinstance(eos, int):
            eos = [eos]
        if raw.get("use_sliding_window", False):
            raise ConfigError(
                "config.json sets use_sliding_window; this architecture's attention is full "
                "and causal in every layer, a windowed variant is not defined for it here"
            )
        if raw.get("rope_scaling") not in (None, {}):
            raise ConfigError(
                f"config.json sets rope_scaling={raw['rope_scaling']!r}; only unscaled rotary "
                "positions are implemented for this architecture"
            )
        if raw.get("hidden_act", "silu") != "silu":
            raise ConfigError(
                f"config.json sets hidden_act={raw['hidden_act']!r}; this architecture's "
                "feed-forward is SiLU-gated"
            )
        cfg = cls(
            hidden_size=hidden,
            intermediate_size=int(_require(raw, "intermediate_size")),
            num_hidden_layers=int(_require(raw, "num_hidden_layers")),
            num_attention_heads=heads,
            num_key_value_heads=int(raw.get("num_key_value_heads", heads)),
            head_dim=int(raw.get("head_dim") or hidden // heads),
            vocab_size=int(_require(raw, "vocab_size")),
            rms_norm_eps=float(raw.get("rms_norm_eps", 1e-6)),
            rope_theta=float(raw.get("rope_theta", 10000.0)),
            max_position_embeddings=int(raw.get("max_position_embeddings", 32768)),
            tie_word_embeddings=bool(raw.get("tie_word_embeddings", False)),
            eos_token_ids=tuple(int(t) for t in eos),
            bos_token_id=raw.get("bos_token_id"),
            architecture=arch,
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        for name in (
            "hidden_size",
            "intermediate_size",
            "num_hidden_layers",
            "num_attention_heads",
            "num_key_value_heads",
            "head_dim",
            "vocab_size",
            "max_position_embeddings",
        ):
            if getattr(self, name) <= 0:
                raise ConfigError(f"{name} must be positive, got {getattr(self, name)}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"num_attention_heads ({self.num_attention_heads}) is not a multiple of "
                f"num_key_value_heads ({self.num_key_value_heads})"
            )
        if self.head_dim % 2:
            raise ConfigError(f"head_dim ({self.head_dim}) must be even for rotary positions")
        if not self.rms_norm_eps > 0:
            raise ConfigError("rms_norm_eps must be positive")

    def to_dict(self) -> dict:
        """The ``config.json`` that reads back to this configuration."""
        out = {
            "architectures": [self.architecture],
            "model_type": "qwen2",
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "vocab_size": self.vocab_size,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "max_position_embeddings": self.max_position_embeddings,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": "silu",
            "use_sliding_window": False,
        }
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        if self.bos_token_id is not None:
            out["bos_token_id"] = self.bos_token_id
        return out

    def kv_bytes_per_token(self, elem_bytes: int = 2) -> int:
        """Bytes of keys and values one token occupies over all layers
        (reference: mercury/config.py:73-81)."""
        return (
            2 * self.num_hidden_layers * self.num_key_value_heads * self.head_dim * elem_bytes
        )


@dataclass(frozen=True)
class LatentMixerConfig:
    """Sizes and constants of one latent-attention mixer (``layers[i].mixer``)."""

    heads: int
    dim: int          # unrotated query/key dims per head
    rot_dim: int      # rotated query/key dims per head (the key's are shared by the heads)
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot_base: float
    rot_dims: int     # how many of the rotated part's dims turn

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "LatentMixerConfig":
        need = lambda key: _require_in(raw, key, where)
        rot = raw.get("rot") or {}
        rot_dim = int(need("rot_dim"))
        dim = int(need("dim"))
        cfg = cls(
            heads=int(need("heads")), dim=dim, rot_dim=rot_dim, vdim=int(need("vdim")),
            q_rank=int(need("q_rank")), kv_rank=int(need("kv_rank")),
            scale=float(raw["scale"]) if raw.get("scale") is not None else (dim + rot_dim) ** -0.5,
            rot_base=float(rot.get("base", 10000.0)),
            rot_dims=int(rot.get("dims", rot_dim)),
        )
        for name in ("heads", "dim", "vdim", "q_rank", "kv_rank"):
            if getattr(cfg, name) <= 0:
                raise ConfigError(f"{where}.{name} must be positive, got {getattr(cfg, name)}")
        if cfg.rot_dim < 0 or cfg.rot_dims < 0 or cfg.rot_dims > cfg.rot_dim or cfg.rot_dims % 2:
            raise ConfigError(f"{where}: {cfg.rot_dims} rotated dims (even) of a rotated part of {cfg.rot_dim}")
        if cfg.rot_dims and not cfg.rot_base > 0:
            raise ConfigError(f"{where}.rot.base must be positive")
        return cfg

    def to_dict(self) -> dict:
        return {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim,
                "q_rank": self.q_rank, "kv_rank": self.kv_rank, "scale": self.scale,
                "rot": {"base": self.rot_base, "dims": self.rot_dims}}


@dataclass(frozen=True)
class FeedForwardConfig:
    """``layers[i].mlp``: a dense gated feed-forward (`experts` 0) or routed experts."""

    ff: int
    limit: float
    experts: int = 0
    top: int = 0
    router_scale: float = 1.0

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "FeedForwardConfig":
        kind = _require_in(raw, "kind", where)
        if kind == "dense":
            cfg = cls(ff=int(_require_in(raw, "ff", where)), limit=float(_require_in(raw, "limit", where)))
        elif kind == "moe":
            expert = _require_in(raw, "expert", where)
            router = _require_in(raw, "router", where)
            cfg = cls(ff=int(_require_in(expert, "ff", where + ".expert")),
                      limit=float(_require_in(expert, "limit", where + ".expert")),
                      experts=int(_require_in(router, "experts", where + ".router")),
                      top=int(_require_in(router, "top", where + ".router")),
                      router_scale=float(router.get("scale", 1.0)))
            if not 0 < cfg.top <= cfg.experts:
                raise ConfigError(f"{where}: top {cfg.top} of {cfg.experts} experts")
        else:
            raise ConfigError(f"{where}.kind {kind!r} is not implemented; known: dense, moe")
        if cfg.ff <= 0 or not cfg.limit > 0:
            raise ConfigError(f"{where}: ff and limit must be positive")
        return cfg

    def to_dict(self) -> dict:
        if not self.experts:
            return {"kind": "dense", "ff": self.ff, "limit": self.limit}
        return {"kind": "moe", "expert": {"ff": self.ff, "limit": self.limit},
                "router": {"experts": self.experts, "top": self.top, "scale": self.router_scale}}


@dataclass(frozen=True)
class TalolornLayerConfig:
    mixer: LatentMixerConfig
    mlp: FeedForwardConfig | None
    weights_of: int | None = None     # the layer whose tensors this one uses


def _require_in(raw: dict, key: str, where: str):
    if not isinstance(raw, dict) or key not in raw:
        raise ConfigError(f"config.json has no {where}.{key}")
    return raw[key]


@dataclass(frozen=True)
class TalolornConfig:
    """The Talolorn decoder: a scaled embedding; layers of one RMS norm whose output a
    latent-attention mixer and a feed-forward (dense or routed experts, or none) both read,
    their sum entering the residual stream times ``residual_mult``; a final RMS norm and an
    untied head.  ``layers`` lists the layers in order; one with ``weights_of: j`` runs layer
    j's tensors over a cache of its own."""

    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    residual_mult: float
    layers: tuple
    architecture: str = "Talolorn"
    eos_token_ids: tuple = ()

    @classmethod
    def from_dict(cls, raw: dict) -> "TalolornConfig":
        entries = _require(raw, "layers")
        if not isinstance(entries, list) or not entries:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers = []
        for i, entry in enumerate(entries):
            where = f"layers[{i}]"
            kind = _require_in(entry, "type", where)
            if kind != "latent_attention":
                raise ConfigError(f"{where}.type {kind!r} is not implemented; known: latent_attention")
            mlp = entry.get("mlp")
            shared = entry.get("weights_of")
            layers.append(TalolornLayerConfig(
                mixer=LatentMixerConfig.from_dict(_require_in(entry, "mixer", where), where + ".mixer"),
                mlp=None if mlp is None else FeedForwardConfig.from_dict(mlp, where + ".mlp"),
                weights_of=None if shared is None else int(shared)))
        cfg = cls(
            vocab=int(_require(raw, "vocab")), width=int(_require(raw, "width")),
            embedding_scale=float((raw.get("embedding") or {}).get("scale", 1.0)),
            norm_eps=float(_require_in(_require(raw, "norm"), "eps", "norm")),
            residual_mult=float(raw.get("residual_mult", 1.0)),
            layers=tuple(layers),
            architecture=str(raw.get("architecture") or (raw.get("architectures") or ["Talolorn"])[0]),
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError("vocab and width must be positive")
        if not self.norm_eps > 0:
            raise ConfigError("norm.eps must be positive")
        for i, layer in enumerate(self.layers):
            j = layer.weights_of
            if j is None:
                continue
            if not 0 <= j < len(self.layers) or self.layers[j].weights_of is not None:
                raise ConfigError(f"layers[{i}].weights_of names {j}, which is no layer with tensors of its own")
            # the layer runs as layer j is described (mixer, feed-forward, norm); the rest of
            # its own entry repeats layer j's

    def to_dict(self) -> dict:
        layers = []
        for layer in self.layers:
            entry = {"type": "latent_attention", "mixer": layer.mixer.to_dict(),
                     "mlp": None if layer.mlp is None else layer.mlp.to_dict()}
            if layer.weights_of is not None:
                entry["weights_of"] = layer.weights_of
            layers.append(entry)
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps},
                "residual_mult": self.residual_mult, "layers": layers}


@dataclass(frozen=True)
class RotatedAttentionConfig:
    """``layers[i].mixer`` of a layer of type ``attention`` (and, with other options, the left
    half of a ``parallel`` one): grouped-query attention whose options are all data."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_base: float = 10000.0
    rot_dims: int = 0            # 0: queries and keys do not turn
    softcap: float = 0.0         # 0: the score is not bounded
    q_temp_coef: float = 0.0
    q_temp_every: int = 0        # 0: no query temperature

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "RotatedAttentionConfig":
        need = lambda key: _require_in(raw, key, where)
        rot = raw.get("rot") or {}
        temp = raw.get("q_temp") or {}
        dim = int(need("dim"))
        cfg = cls(
            heads=int(need("heads")), kv_heads=int(need("kv_heads")), dim=dim,
            vdim=int(raw.get("vdim", dim)), scale=float(need("scale")),
            rot_base=float(rot.get("base", 10000.0)), rot_dims=int(rot.get("dims", 0)),
            softcap=float(raw.get("softcap") or 0.0),
            q_temp_coef=float(temp.get("coef", 0.0)), q_temp_every=int(temp.get("every", 0)))
        for name in ("heads", "kv_heads", "dim", "vdim"):
            if getattr(cfg, name) <= 0:
                raise ConfigError(f"{where}.{name} must be positive, got {getattr(cfg, name)}")
        if cfg.heads % cfg.kv_heads:
            raise ConfigError(f"{where}: {cfg.heads} heads are not a multiple of {cfg.kv_heads} kv_heads")
        if cfg.rot_dims < 0 or cfg.rot_dims > cfg.dim or cfg.rot_dims % 2:
            raise ConfigError(f"{where}.rot.dims {cfg.rot_dims} must be even and within dim {cfg.dim}")
        if cfg.rot_dims and not cfg.rot_base > 0:
            raise ConfigError(f"{where}.rot.base must be positive")
        if cfg.softcap < 0 or cfg.q_temp_every < 0:
            raise ConfigError(f"{where}: softcap and q_temp.every are not negative")
        return cfg

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
               "scale": self.scale}
        if self.rot_dims:
            out["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
        if self.softcap:
            out["softcap"] = self.softcap
        if self.q_temp_every:
            out["q_temp"] = {"coef": self.q_temp_coef, "every": self.q_temp_every}
        return out


@dataclass(frozen=True)
class StateSpaceConfig:
    """The right half of a ``parallel`` mixer: a state-space mixer's sizes."""

    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "StateSpaceConfig":
        need = lambda key: int(_require_in(raw, key, where))
        cfg = cls(heads=need("heads"), vdim=need("vdim"), state=need("state"), groups=need("groups"),
                  conv=need("conv"), norm_groups=int(raw.get("norm_groups", 1)))
        for name in ("heads", "vdim", "state", "groups", "conv", "norm_groups"):
            if getattr(cfg, name) <= 0:
                raise ConfigError(f"{where}.{name} must be positive, got {getattr(cfg, name)}")
        if cfg.heads % cfg.groups:
            raise ConfigError(f"{where}: {cfg.heads} heads are not a multiple of {cfg.groups} groups")
        if (cfg.heads * cfg.vdim) % cfg.norm_groups:
            raise ConfigError(f"{where}: heads * vdim does not split into {cfg.norm_groups} norm_groups")
        return cfg

    def to_dict(self) -> dict:
        return {"heads": self.heads, "vdim": self.vdim, "state": self.state, "groups": self.groups,
                "conv": self.conv, "norm_groups": self.norm_groups}


@dataclass(frozen=True)
class LarozenLayerConfig:
    kind: str                 # "attention" or "parallel"
    attention: RotatedAttentionConfig     # the mixer, or the left half of a parallel one
    state_space: StateSpaceConfig | None  # the right half of a parallel one
    ff: int                   # 0: no feed-forward


@dataclass(frozen=True)
class LarozenConfig:
    """The Larozen decoder: pre-norm layers (RMS norms whose stored weight lies around zero)
    over a float32 stream; a layer's mixer is either a rotated grouped-query attention with a
    bounded score whose values are its keys, or a sink attention and a state-space mixer side
    by side; the feed-forward is down(relu(up(x))^2) or absent; the head is the embedding.
    ``loop`` runs layers start .. stop - 1 `times` times in a row with the same tensors, every
    pass over a cache and state of its own, the stream re-entering each pass through a
    projection of itself beside the embedding output."""

    vocab: int
    width: int
    norm_eps: float
    layers: tuple
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1       # loop_stop == loop_start: no loop
    architecture: str = "Larozen"
    eos_token_ids: tuple = ()

    @property
    def loops(self) -> bool:
        return self.loop_stop > self.loop_start

    def order(self) -> list:
        """(layer, whether the stream re-enters before it) in the order the layers run."""
        n = len(self.layers)
        if not self.loops:
            return [(i, False) for i in range(n)]
        out = [(i, False) for i in range(self.loop_start)]
        for _ in range(self.loop_times):
            out += [(i, i == self.loop_start) for i in range(self.loop_start, self.loop_stop)]
        return out + [(i, False) for i in range(self.loop_stop, n)]

    @classmethod
    def from_dict(cls, raw: dict) -> "LarozenConfig":
        entries = _require(raw, "layers")
        if not isinstance(entries, list) or not entries:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers = []
        for i, entry in enumerate(entries):
            where = f"layers[{i}]"
            kind = _require_in(entry, "type", where)
            mixer = _require_in(entry, "mixer", where)
            if kind == "attention":
                attention = RotatedAttentionConfig.from_dict(mixer, where + ".mixer")
                if attention.vdim != attention.dim:
                    raise ConfigError(f"{where}.mixer: the values are the keys, so vdim is dim")
                state_space = None
            elif kind == "parallel":
                attention = RotatedAttentionConfig.from_dict(
                    _require_in(mixer, "left", where + ".mixer"), where + ".mixer.left")
                state_space = StateSpaceConfig.from_dict(
                    _require_in(mixer, "right", where + ".mixer"), where + ".mixer.right")
            else:
                raise ConfigError(f"{where}.type {kind!r} is not implemented; known: attention, parallel")
            mlp = entry.get("mlp")
            ff = 0
            if mlp is not None:
                if _require_in(mlp, "kind", where + ".mlp") != "dense":
                    raise ConfigError(f"{where}.mlp.kind {mlp['kind']!r} is not implemented; known: dense")
                ff = int(_require_in(mlp, "ff", where + ".mlp"))
                if ff <= 0:
                    raise ConfigError(f"{where}.mlp.ff must be positive")
            layers.append(LarozenLayerConfig(kind, attention, state_space, ff))
        loop = raw.get("loop") or {}
        cfg = cls(
            vocab=int(_require(raw, "vocab")), width=int(_require(raw, "width")),
            norm_eps=float(_require_in(_require(raw, "norm"), "eps", "norm")),
            layers=tuple(layers),
            loop_start=int(loop.get("start", 0)), loop_stop=int(loop.get("stop", 0)) if loop else 0,
            loop_times=int(loop.get("times", 1)),
            architecture=str(raw.get("architecture") or (raw.get("architectures") or ["Larozen"])[0]),
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError("vocab and width must be positive")
        if not self.norm_eps > 0:
            raise ConfigError("norm.eps must be positive")
        if self.loops or self.loop_times != 1:
            if not 0 <= self.loop_start < self.loop_stop <= len(self.layers) or self.loop_times < 1:
                raise ConfigError(f"loop: layers {self.loop_start} .. {self.loop_stop} - 1, "
                                  f"{self.loop_times} times, of {len(self.layers)} layers")

    def to_dict(self) -> dict:
        layers = []
        for layer in self.layers:
            mixer = layer.attention.to_dict()
            if layer.kind == "parallel":
                mixer = {"left": mixer, "right": layer.state_space.to_dict()}
            layers.append({"type": layer.kind, "mixer": mixer,
                           "mlp": {"kind": "dense", "ff": layer.ff} if layer.ff else None})
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
               "norm": {"eps": self.norm_eps}, "layers": layers}
        if self.loops:
            out["loop"] = {"start": self.loop_start, "stop": self.loop_stop, "times": self.loop_times}
        return out


@dataclass(frozen=True)
class DifferentialAttentionConfig:
    """``layers[i].mixer`` of a Videdra layer of type ``attention``: grouped-query differential
    attention (two score maps a head over the same values), a window that keeps the
    sequence's first tokens, a gate per head; with ``kv_from`` the layer owns no key and value
    projections and reads the cache of the layer named."""

    heads: int
    kv_heads: int
    dim: int                 # per map
    vdim: int
    scale: float
    diff: float
    window: int = 0          # 0: every earlier token
    keep_first: int = 0
    rot_base: float = 10000.0
    rot_dims: int = 0        # 0: queries and keys do not turn
    kv_from: int | None = None

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "DifferentialAttentionConfig":
        need = lambda key: _require_in(raw, key, where)
        rot = raw.get("rot") or {}
        mask = raw.get("mask") or {}
        dim = int(need("dim"))
        source = raw.get("kv_from")
        cfg = cls(
            heads=int(need("heads")), kv_heads=int(need("kv_heads")), dim=dim,
            vdim=int(raw.get("vdim", dim)), scale=float(need("scale")), diff=float(need("diff")),
            window=int(mask.get("size") or 0), keep_first=int(mask.get("keep_first") or 0),
            rot_base=float(rot.get("base", 10000.0)), rot_dims=int(rot.get("dims", 0)),
            kv_from=None if source is None else int(source))
        for name in ("heads", "kv_heads", "dim", "vdim"):
            if getattr(cfg, name) <= 0:
                raise ConfigError(f"{where}.{name} must be positive, got {getattr(cfg, name)}")
        if cfg.heads % cfg.kv_heads:
            raise ConfigError(f"{where}: {cfg.heads} heads are not a multiple of {cfg.kv_heads} kv_heads")
        if cfg.rot_dims < 0 or cfg.rot_dims > cfg.dim or cfg.rot_dims % 2:
            raise ConfigError(f"{where}.rot.dims {cfg.rot_dims} must be even and within dim {cfg.dim}")
        if cfg.rot_dims and not cfg.rot_base > 0:
            raise ConfigError(f"{where}.rot.base must be positive")
        if cfg.window < 0 or cfg.keep_first < 0:
            raise ConfigError(f"{where}.mask: size and keep_first are not negative")
        return cfg

    def same_cache_as(self, other: "DifferentialAttentionConfig") -> bool:
        """Whether keys and values the other layer stores are what this one would store."""
        mine = (self.heads, self.kv_heads, self.dim, self.vdim, self.rot_dims,
                self.rot_base if self.rot_dims else 0.0)
        theirs = (other.heads, other.kv_heads, other.dim, other.vdim, other.rot_dims,
                  other.rot_base if other.rot_dims else 0.0)
        return mine == theirs

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
               "scale": self.scale, "diff": self.diff}
        if self.window:
            out["mask"] = {"size": self.window, "keep_first": self.keep_first}
        if self.rot_dims:
            out["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
        if self.kv_from is not None:
            out["kv_from"] = self.kv_from
        return out


@dataclass(frozen=True)
class RetentionConfig:
    """``layers[i].mixer`` of a Videdra layer of type ``retention``."""

    heads: int
    dim: int
    vdim: int
    decay: tuple
    rot_base: float = 10000.0
    rot_dims: int = 0

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "RetentionConfig":
        need = lambda key: _require_in(raw, key, where)
        rot = raw.get("rot") or {}
        dim = int(need("dim"))
        cfg = cls(heads=int(need("heads")), dim=dim, vdim=int(raw.get("vdim", dim)),
                  decay=tuple(float(g) for g in need("decay")),
                  rot_base=float(rot.get("base", 10000.0)), rot_dims=int(rot.get("dims", 0)))
        for name in ("heads", "dim", "vdim"):
            if getattr(cfg, name) <= 0:
                raise ConfigError(f"{where}.{name} must be positive, got {getattr(cfg, name)}")
        if len(cfg.decay) != cfg.heads:
            raise ConfigError(f"{where}.decay lists {len(cfg.decay)} values for {cfg.heads} heads")
        if any(not 0.0 <= g <= 1.0 for g in cfg.decay):
            raise ConfigError(f"{where}.decay: every head's decay lies in [0, 1]")
        if cfg.rot_dims < 0 or cfg.rot_dims > cfg.dim or cfg.rot_dims % 2:
            raise ConfigError(f"{where}.rot.dims {cfg.rot_dims} must be even and within dim {cfg.dim}")
        if cfg.rot_dims and not cfg.rot_base > 0:
            raise ConfigError(f"{where}.rot.base must be positive")
        return cfg

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "decay": list(self.decay)}
        if self.rot_dims:
            out["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
        return out


@dataclass(frozen=True)
class VidedraMlpConfig:
    """``layers[i].mlp``: ``dense`` (one gated feed-forward of `ff`) or ``moe`` (`experts`
    gated feed-forwards of `ff` of which a token uses `top`, and a shared one of `shared_ff`
    when that is not 0)."""

    kind: str
    ff: int
    experts: int = 0
    top: int = 0
    shared_ff: int = 0

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "VidedraMlpConfig":
        kind = _require_in(raw, "kind", where)
        if kind == "dense":
            cfg = cls("dense", int(_require_in(raw, "ff", where)))
        elif kind == "moe":
            router = _require_in(raw, "router", where)
            shared = raw.get("shared")
            cfg = cls("moe", int(_require_in(_require_in(raw, "expert", where), "ff", where + ".expert")),
                      experts=int(_require_in(router, "experts", where + ".router")),
                      top=int(_require_in(router, "top", where + ".router")),
                      shared_ff=int(_require_in(shared, "ff", where + ".shared")) if shared else 0)
            if not 0 < cfg.top <= cfg.experts:
                raise ConfigError(f"{where}.router: top {cfg.top} of {cfg.experts} experts")
            if shared and cfg.shared_ff <= 0:
                raise ConfigError(f"{where}.shared.ff must be positive")
        else:
            raise ConfigError(f"{where}.kind {kind!r} is not implemented; known: dense, moe")
        if cfg.ff <= 0:
            raise ConfigError(f"{where}: ff must be positive")
        return cfg

    def to_dict(self) -> dict:
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        out = {"kind": "moe", "expert": {"ff": self.ff},
               "router": {"experts": self.experts, "top": self.top}}
        if self.shared_ff:
            out["shared"] = {"ff": self.shared_ff}
        return out


@dataclass(frozen=True)
class VidedraLayerConfig:
    kind: str                                   # "attention" or "retention"
    mixer: object                               # DifferentialAttentionConfig | RetentionConfig
    mlp: VidedraMlpConfig | None


@dataclass(frozen=True)
class VidedraConfig:
    """The Videdra decoder: layers with an RMS norm before and after each sublayer and a stored
    vector per channel on what enters the float32 stream; a layer's mixer is a differential
    attention (which may read an earlier layer's keys and values) or a retention with
    per-request state; its feed-forward a tanh-gelu gated one, routed SiLU experts with a gated
    shared expert, or none; an untied head behind a final norm."""

    vocab: int
    width: int
    norm_eps: float
    layers: tuple
    architecture: str = "Videdra"
    eos_token_ids: tuple = ()

    @classmethod
    def from_dict(cls, raw: dict) -> "VidedraConfig":
        entries = _require(raw, "layers")
        if not isinstance(entries, list) or not entries:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers = []
        for i, entry in enumerate(entries):
            where = f"layers[{i}]"
            kind = _require_in(entry, "type", where)
            mixer = _require_in(entry, "mixer", where)
            if kind == "attention":
                mixer_cfg = DifferentialAttentionConfig.from_dict(mixer, where + ".mixer")
            elif kind == "retention":
                mixer_cfg = RetentionConfig.from_dict(mixer, where + ".mixer")
            else:
                raise ConfigError(f"{where}.type {kind!r} is not implemented; known: attention, retention")
            mlp = entry.get("mlp")
            layers.append(VidedraLayerConfig(
                kind, mixer_cfg, None if mlp is None else VidedraMlpConfig.from_dict(mlp, where + ".mlp")))
        cfg = cls(vocab=int(_require(raw, "vocab")), width=int(_require(raw, "width")),
                  norm_eps=float(_require_in(_require(raw, "norm"), "eps", "norm")),
                  layers=tuple(layers),
                  architecture=str(raw.get("architecture") or (raw.get("architectures") or ["Videdra"])[0]))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError("vocab and width must be positive")
        if not self.norm_eps > 0:
            raise ConfigError("norm.eps must be positive")
        for i, layer in enumerate(self.layers):
            source = getattr(layer.mixer, "kv_from", None)
            if source is None:
                continue
            where = f"layers[{i}].mixer.kv_from"
            if not 0 <= source < i:
                raise ConfigError(f"{where} {source} names no earlier layer")
            other = self.layers[source]
            if other.kind != "attention" or other.mixer.kv_from is not None:
                raise ConfigError(f"{where}: layer {source} projects no keys and values of its own")
            if not layer.mixer.same_cache_as(other.mixer):
                raise ConfigError(f"{where}: layer {source} has other head counts, sizes or rotation")

    def to_dict(self) -> dict:
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                "norm": {"eps": self.norm_eps},
                "layers": [{"type": layer.kind, "mixer": layer.mixer.to_dict(),
                            "mlp": None if layer.mlp is None else layer.mlp.to_dict()}
                           for layer in self.layers]}


def _rotation(raw: dict, where: str, width: int) -> tuple:
    """(base, dims, scaling) of a mixer's ``rot`` entry; dims 0 when there is none.  `scaling`
    is None or (factor, low, high, original)."""
    rot = raw.get("rot") or {}
    dims = int(rot.get("dims", 0))
    base = float(rot.get("base", 10000.0))
    if dims < 0 or dims > width or dims % 2:
        raise ConfigError(f"{where}.rot.dims {dims} must be even and within {width}")
    if dims and not base > 0:
        raise ConfigError(f"{where}.rot.base must be positive")
    s = rot.get("scaling")
    scaling = None
    if s:
        at = where + ".rot.scaling"
        scaling = tuple(float(_require_in(s, key, at)) for key in ("factor", "low", "high", "original"))
        factor, low, high, original = scaling
        if not (factor > 0 and high > low >= 0 and original > 0):
            raise ConfigError(f"{at}: factor > 0, high > low >= 0 and original > 0 are required")
    return base, dims, scaling


def _rotation_dict(base: float, dims: int, scaling) -> dict:
    out = {"base": base, "dims": dims}
    if scaling:
        out["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return out


@dataclass(frozen=True)
class GatedAttentionConfig:
    """``layers[i].mixer`` of a Mogilorn layer of type ``attention``: grouped-query causal
    attention with biased projections, a norm per query and key head, interleaved rotation whose
    frequencies may be scaled, a bounded score, values that may be mixed with the first such
    layer's, and a sigmoid gate per output column."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float = 0.0       # 0: the score is not bounded
    v_mix: bool = False
    rot_base: float = 10000.0
    rot_dims: int = 0          # 0: queries and keys do not turn
    rot_scaling: tuple | None = None

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "GatedAttentionConfig":
        need = lambda key: _require_in(raw, key, where)
        dim = int(need("dim"))
        base, dims, scaling = _rotation(raw, where, dim)
        cfg = cls(heads=int(need("heads")), kv_heads=int(raw.get("kv_heads") or need("heads")),
                  dim=dim, vdim=int(raw.get("vdim") or dim), scale=float(need("scale")),
                  softcap=float(raw.get("softcap") or 0.0), v_mix=bool(raw.get("v_mix", False)),
                  rot_base=base, rot_dims=dims, rot_scaling=scaling)
        for name in ("heads", "kv_heads", "dim", "vdim"):
            if getattr(cfg, name) <= 0:
                raise ConfigError(f"{where}.{name} must be positive, got {getattr(cfg, name)}")
        if cfg.heads % cfg.kv_heads:
            raise ConfigError(f"{where}: {cfg.heads} heads are not a multiple of {cfg.kv_heads} kv_heads")
        if cfg.softcap < 0:
            raise ConfigError(f"{where}.softcap is not negative")
        return cfg

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
               "scale": self.scale, "v_mix": self.v_mix}
        if self.softcap:
            out["softcap"] = self.softcap
        if self.rot_dims:
            out["rot"] = _rotation_dict(self.rot_base, self.rot_dims, self.rot_scaling)
        return out


@dataclass(frozen=True)
class MatrixMemoryConfig:
    """``layers[i].mixer`` of a Mogilorn layer of type ``mlstm``."""

    heads: int
    dim: int
    vdim: int
    gate_cap: float = 0.0      # 0: the gates' logits are not bounded

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "MatrixMemoryConfig":
        need = lambda key: _require_in(raw, key, where)
        dim = int(need("dim"))
        cfg = cls(heads=int(need("heads")), dim=dim, vdim=int(raw.get("vdim") or dim),
                  gate_cap=float(raw.get("gate_cap") or 0.0))
        for name in ("heads", "dim", "vdim"):
            if getattr(cfg, name) <= 0:
                raise ConfigError(f"{where}.{name} must be positive, got {getattr(cfg, name)}")
        if cfg.gate_cap < 0:
            raise ConfigError(f"{where}.gate_cap is not negative")
        return cfg

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim}
        if self.gate_cap:
            out["gate_cap"] = self.gate_cap
        return out


@dataclass(frozen=True)
class WindowedLatentConfig:
    """``layers[i].mixer`` of a Mogilorn layer of type ``latent_attention``: attention through
    a normed latent and one rotated key part shared by the heads, queries straight from the
    input, a sliding window, a sink per head and a sigmoid gate per output column."""

    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    window: int = 0            # 0: every earlier token
    rot_base: float = 10000.0
    rot_dims: int = 0
    rot_scaling: tuple | None = None

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "WindowedLatentConfig":
        need = lambda key: _require_in(raw, key, where)
        rot_dim = int(raw.get("rot_dim") or 0)
        base, dims, scaling = _rotation(raw, where, rot_dim)
        if raw.get("rot") is not None and "dims" not in raw["rot"]:
            dims = rot_dim - rot_dim % 2
        cfg = cls(heads=int(need("heads")), dim=int(need("dim")), rot_dim=rot_dim,
                  vdim=int(need("vdim")), kv_rank=int(need("kv_rank")), scale=float(need("scale")),
                  window=int((raw.get("mask") or {}).get("size") or 0),
                  rot_base=base, rot_dims=dims, rot_scaling=scaling)
        for name in ("heads", "dim", "vdim", "kv_rank"):
            if getattr(cfg, name) <= 0:
                raise ConfigError(f"{where}.{name} must be positive, got {getattr(cfg, name)}")
        if cfg.rot_dim < 0 or cfg.window < 0:
            raise ConfigError(f"{where}: rot_dim and mask.size are not negative")
        return cfg

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim,
               "kv_rank": self.kv_rank, "scale": self.scale}
        if self.window:
            out["mask"] = {"size": self.window}
        if self.rot_dims:
            out["rot"] = _rotation_dict(self.rot_base, self.rot_dims, self.rot_scaling)
        return out


@dataclass(frozen=True)
class MogilornLayerConfig:
    kind: str                  # "attention", "mlstm" or "latent_attention"
    mixer: object
    ff: int                    # 0: the layer has no feed-forward


MOGILORN_MIXERS = {"attention": GatedAttentionConfig, "mlstm": MatrixMemoryConfig,
                   "latent_attention": WindowedLatentConfig}


@dataclass(frozen=True)
class MogilornConfig:
    """The Mogilorn decoder: a scaled embedding; layers whose sublayers read the float32 stream
    itself and whose outputs are RMS-normed (weights stored around zero) before they enter
    it; a mixer per layer out of a gated grouped-query attention, a matrix memory with
    per-request state and a windowed latent attention with sinks; a tanh-gelu feed-forward or
    none; the head is the embedding, behind a final norm."""

    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float
    layers: tuple
    architecture: str = "Mogilorn"
    eos_token_ids: tuple = ()

    @classmethod
    def from_dict(cls, raw: dict) -> "MogilornConfig":
        entries = _require(raw, "layers")
        if not isinstance(entries, list) or not entries:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers = []
        for i, entry in enumerate(entries):
            where = f"layers[{i}]"
            kind = _require_in(entry, "type", where)
            if kind not in MOGILORN_MIXERS:
                raise ConfigError(f"{where}.type {kind!r} is not implemented; known: "
                                  f"{', '.join(sorted(MOGILORN_MIXERS))}")
            mixer = MOGILORN_MIXERS[kind].from_dict(_require_in(entry, "mixer", where), where + ".mixer")
            mlp, ff = entry.get("mlp"), 0
            if mlp is not None:
                if _require_in(mlp, "kind", where + ".mlp") != "dense":
                    raise ConfigError(f"{where}.mlp.kind {mlp['kind']!r} is not implemented; known: dense")
                ff = int(_require_in(mlp, "ff", where + ".mlp"))
                if ff <= 0:
                    raise ConfigError(f"{where}.mlp.ff must be positive")
            layers.append(MogilornLayerConfig(kind, mixer, ff))
        cfg = cls(vocab=int(_require(raw, "vocab")), width=int(_require(raw, "width")),
                  norm_eps=float(_require_in(_require(raw, "norm"), "eps", "norm")),
                  embedding_scale=float((raw.get("embedding") or {}).get("scale", 1.0)),
                  layers=tuple(layers),
                  architecture=str(raw.get("architecture") or (raw.get("architectures") or ["Mogilorn"])[0]))
        cfg.validate()
        return cfg

    def mixing_layers(self) -> list:
        """Indices of the attention layers whose values are mixed, the first one first."""
        return [i for i, layer in enumerate(self.layers)
                if layer.kind == "attention" and layer.mixer.v_mix]

    def validate(self) -> None:
        if self.vocab <= 0 or self.width <= 0:
            raise ConfigError("vocab and width must be positive")
        if not self.norm_eps > 0:
            raise ConfigError("norm.eps must be positive")
        mixing = self.mixing_layers()
        for i in mixing[1:]:
            first, m = self.layers[mixing[0]].mixer, self.layers[i].mixer
            # (the blend runs over a token's value columns side by side: as many are needed)
            if m.kv_heads * m.vdim != first.kv_heads * first.vdim:
                raise ConfigError(f"layers[{i}].mixer mixes its values with layer {mixing[0]}'s, "
                                  "which has another number of value columns (kv_heads * vdim)")

    def to_dict(self) -> dict:
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                "norm": {"eps": self.norm_eps}, "embedding": {"scale": self.embedding_scale},
                "layers": [{"type": layer.kind, "mixer": layer.mixer.to_dict(),
                            "mlp": {"kind": "dense", "ff": layer.ff} if layer.ff else None}
                           for layer in self.layers]}
