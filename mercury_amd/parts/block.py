"""How a layer's parts are arranged around the residual stream."""

from __future__ import annotations

from ..hostcore import core
from ..kernels import ops
from .base import FeedForward, Mixer, Norm, Part
from .lowering import OneOp


class PreNormBlock(Part):
    """h += mixer(norm_1(h)); h += ffn(norm_2(h)), h being the float32 residual stream.

    This is the reference's layer (mercury/model/qwen2.py:82-94) with its carried `residual`
    written as the running sum: the reference adds the previous output inside the next norm,
    here each part adds its output into h as it produces it.

    `names` gives the checkpoint sub-prefix of each part, e.g. ``{"mixer": "self_attn.",
    "ffn": "mlp.", "norm_mixer": "input_layernorm.", "norm_ffn": "post_attention_layernorm."}``.
    """

    def __init__(self, mixer: Mixer, ffn: FeedForward | None, norm_mixer: Norm,
                 norm_ffn: Norm | None, names: dict):
        self.mixer, self.ffn, self.norm_mixer, self.norm_ffn = mixer, ffn, norm_mixer, norm_ffn
        self.names = dict(names)

    def _children(self):
        out = [("mixer", self.mixer), ("norm_mixer", self.norm_mixer)]
        if self.ffn is not None:
            out += [("ffn", self.ffn), ("norm_ffn", self.norm_ffn)]
        return out

    @property
    def graph_safe(self) -> bool:
        return all(part.graph_safe for _, part in self._children())

    def lowerable_with(self, state) -> bool:
        """Whether the host core can run the whole layer: every part hands over its work, and
        a mixer with state of its own says that its operations take the state tensor
        (`lowers_state`)."""
        if state is not None and not getattr(self.mixer, "lowers_state", False):
            return False
        return all(part.can_lower() for _, part in self._children())

    def lower(self, program, cache, state=None) -> None:
        self.norm_mixer.lower(program)
        if state is None:
            self.mixer.lower(program, cache)
        else:
            self.mixer.lower(program, cache, state)
        if self.ffn is not None:
            self.norm_ffn.lower(program)
            self.ffn.lower(program)

    def param_specs(self) -> dict:
        specs = {}
        for key, part in self._children():
            for name, spec in part.param_specs().items():
                specs[self.names[key] + name] = spec
        return specs

    def bind(self, params, dtype, device) -> None:
        for key, part in self._children():
            prefix = self.names[key]
            part.bind({n[len(prefix):]: t for n, t in params.items() if n.startswith(prefix)},
                      dtype, device)

    def prepare(self, max_positions: int, device) -> None:
        self.mixer.prepare(max_positions, device)

    def weight_bytes(self) -> int:
        return sum(part.weight_bytes() for _, part in self._children())

    def forward(self, h, step, cache, state, dtype, pending=None):
        """Runs the layer on the stream h.  `pending` are partial sums [P, T, H] that still
        have to be added into h (the previous projection's, when it left them to its
        consumer); the return value is the same for whoever reads h next."""
        x = self.norm_mixer.forward(h, dtype, partials=pending)
        pending = self.mixer.forward(x, step, cache, state, h)
        if self.ffn is not None:
            x = self.norm_ffn.forward(h, dtype, partials=pending)
            pending = self.ffn.forward(x, step, h)
        return pending


class PrePostNormBlock(Part):
    """A norm before and after each sublayer, and a stored vector per channel on what enters
    the stream:

        h += scale_1 * post_1(mixer(norm_1(h)));   h += scale_2 * post_2(ffn(norm_2(h)))

    with h the float32 residual stream, every norm an :class:`RMSNorm` over the model width
    and scale_i ``<names["scale_mixer"]>`` / ``<names["scale_ffn"]>`` (float32 [hidden]; absent
    when `layer_scale` is off).  `ffn` may be None.  Lowered, a sublayer is its norm and one
    ``post_norm`` operation that holds the sublayer's own operation and runs it over a zeroed
    buffer in the stream's place.  `names` gives the stored sub-prefix of every part:
    ``{"mixer", "ffn", "norm_mixer", "norm_ffn", "post_mixer", "post_ffn", "scale_mixer",
    "scale_ffn"}``.
    """

    def __init__(self, mixer: Mixer, ffn: FeedForward | None, norm_mixer: Norm,
                 norm_ffn: Norm | None, post_mixer: Norm, post_ffn: Norm | None, names: dict,
                 layer_scale: bool = True, stream_given: bool = False,
                 next_reads_stream: bool = False):
        # Sublayers that read the stream itself (a `NoNorm` before them) need it in the compute
        # dtype: the norm behind the sublayer before writes it out with the new stream, where
        # there is one.  `stream_given`: the layer before this one does so for this layer's
        # mixer (built with `next_reads_stream`); both concern the model's program only, a layer
        # that runs alone makes its own copy.
        self.stream_given, self.next_reads_stream = bool(stream_given), bool(next_reads_stream)
        self.mixer, self.ffn = mixer, ffn
        self.norm_mixer, self.norm_ffn = norm_mixer, norm_ffn
        self.post_mixer, self.post_ffn = post_mixer, post_ffn
        self.layer_scale = bool(layer_scale)
        self.names = dict(names)
        self.scale_mixer = self.scale_ffn = None
        self._alone: dict = {}

    def _children(self):
        out = [("mixer", self.mixer), ("norm_mixer", self.norm_mixer), ("post_mixer", self.post_mixer)]
        if self.ffn is not None:
            out += [("ffn", self.ffn), ("norm_ffn", self.norm_ffn), ("post_ffn", self.post_ffn)]
        return out

    def _scales(self):
        if not self.layer_scale:
            return []
        return ["scale_mixer"] + (["scale_ffn"] if self.ffn is not None else [])

    @property
    def graph_safe(self) -> bool:
        return all(part.graph_safe for _, part in self._children())

    def lowerable_with(self, state) -> bool:
        if state is not None and not getattr(self.mixer, "lowers_state", False):
            return False
        return all(part.can_lower() for _, part in self._children())

    def _wrapped(self, program, sub: "_Recorder", post: Norm, scale, gives_x: bool = False) -> None:
        if len(sub.ops) != 1:
            raise ValueError("a sublayer between two norms lowers itself to one operation")
        if getattr(sub, "carried", 0):
            program.need_carried(sub.carried)
        if getattr(post, "one_plus", False) and post.weight is None:
            raise ValueError("the norm behind a sublayer has no weight yet")
        program.append("post_norm", core.post_norm_params(
            sub.ops[0][0], sub.ops[0][1], post.weight.data_ptr(), ops.dtype_code(post.weight.dtype),
            0 if scale is None else scale.data_ptr(), post.eps, gives_x=gives_x))

    def lower(self, program, cache, state=None, alone: bool = False) -> None:
        from .norm import NoNorm

        reads_stream = lambda norm: isinstance(norm, NoNorm)
        if alone or not (self.stream_given and reads_stream(self.norm_mixer)):
            self.norm_mixer.lower(program)
        sub = _Recorder()
        if state is None:
            self.mixer.lower(sub, cache)
        else:
            self.mixer.lower(sub, cache, state)
        hands_on = not alone and self.next_reads_stream
        if self.ffn is None:
            self._wrapped(program, sub, self.post_mixer, self.scale_mixer, gives_x=hands_on)
            return
        within = reads_stream(self.norm_ffn)
        self._wrapped(program, sub, self.post_mixer, self.scale_mixer, gives_x=within)
        if not within:
            self.norm_ffn.lower(program)
        sub = _Recorder()
        self.ffn.lower(sub)
        self._wrapped(program, sub, self.post_ffn, self.scale_ffn, gives_x=hands_on)

    def param_specs(self) -> dict:
        from .base import TensorSpec

        specs = {}
        for key, part in self._children():
            for name, spec in part.param_specs().items():
                specs[self.names[key] + name] = spec
        width = self.post_mixer.size
        for key in self._scales():
            specs[self.names[key]] = TensorSpec((width,), role="vector", init="one_plus_normal")
        return specs

    def bind(self, params, dtype, device) -> None:
        scale_names = {self.names[key] for key in self._scales()}
        for key, part in self._children():
            prefix = self.names[key]
            part.bind({n[len(prefix):]: t for n, t in params.items()
                       if n.startswith(prefix) and n not in scale_names}, dtype, device)
        if self.layer_scale:
            self.scale_mixer = params[self.names["scale_mixer"]].float().contiguous()
            if self.ffn is not None:
                self.scale_ffn = params[self.names["scale_ffn"]].float().contiguous()
        self._alone.clear()

    def prepare(self, max_positions: int, device) -> None:
        self.mixer.prepare(max_positions, device)

    def weight_bytes(self) -> int:
        total = sum(part.weight_bytes() for _, part in self._children())
        return total + sum(t.numel() * 4 for t in (self.scale_mixer, self.scale_ffn) if t is not None)

    def forward(self, h, step, cache, state, dtype, pending=None):
        if not self.lowerable_with(state):
            raise NotImplementedError("a layer with norms behind its sublayers runs as operations "
                                      "of the host core: every part of it must lower itself")
        key = (None if cache is None else cache.k.data_ptr(), None if state is None else state.data_ptr())
        alone = self._alone.get(key)
        if alone is None:
            alone = self._alone[key] = OneOp(
                dtype, h.shape[1], 0, lambda program: self.lower(program, cache, state, alone=True))
        _logits, _x, left = alone.run(step, h, pending=pending)
        return left


class _Recorder:
    """Stands in for a program while a sublayer lowers itself: keeps what it appends."""

    def __init__(self):
        self.ops: list = []

    def append(self, kind: str, params: bytes) -> None:
        self.ops.append((kind, params))

    def need_carried(self, width: int) -> None:
        self.carried = max(getattr(self, "carried", 0), int(width))


class ParallelBlock(Part):
    """h += mult * (mixer(x) + ffn(x)) with x = norm(h): one norm, both sublayers read its
    output, and their sum enters the float32 residual stream scaled by `mult`.  `ffn` may be
    None.

    Lowered, the layer is the norm and one ``parallel`` operation that holds the sublayers'
    own operations (each must lower itself to exactly one) and runs them on the same x, their
    outputs going into a buffer in the stream's place.  `names` gives the checkpoint
    sub-prefix of each part: ``{"mixer": ..., "ffn": ..., "norm": ...}``.
    """

    def __init__(self, mixer: Mixer, ffn: FeedForward | None, norm: Norm, names: dict,
                 residual_mult: float = 1.0):
        self.mixer, self.ffn, self.norm = mixer, ffn, norm
        self.residual_mult = float(residual_mult)
        self.names = dict(names)
        self._alone: dict = {}

    def _children(self):
        out = [("mixer", self.mixer), ("norm", self.norm)]
        if self.ffn is not None:
            out.append(("ffn", self.ffn))
        return out

    @property
    def graph_safe(self) -> bool:
        return all(part.graph_safe for _, part in self._children())

    def lowerable_with(self, state) -> bool:
        if state is not None and not getattr(self.mixer, "lowers_state", False):
            return False
        return all(part.can_lower() for _, part in self._children())

    def lower(self, program, cache, state=None) -> None:
        self.norm.lower(program)
        sub = _Recorder()
        if state is None:
            self.mixer.lower(sub, cache)
        else:
            self.mixer.lower(sub, cache, state)
        if self.ffn is not None:
            self.ffn.lower(sub)
        if len(sub.ops) != (1 if self.ffn is None else 2):
            raise ValueError("a sublayer of a parallel block lowers itself to one operation")
        if getattr(sub, "carried", 0):
            program.need_carried(sub.carried)
        program.append("parallel", core.parallel_params(self.residual_mult, sub.ops))

    def param_specs(self) -> dict:
        specs = {}
        for key, part in self._children():
            for name, spec in part.param_specs().items():
                specs[self.names[key] + name] = spec
        return specs

    def bind(self, params, dtype, device) -> None:
        for key, part in self._children():
            prefix = self.names[key]
            part.bind({n[len(prefix):]: t for n, t in params.items() if n.startswith(prefix)},
                      dtype, device)
        self._alone.clear()

    def prepare(self, max_positions: int, device) -> None:
        self.mixer.prepare(max_positions, device)

    def weight_bytes(self) -> int:
        return sum(part.weight_bytes() for _, part in self._children())

    def forward(self, h, step, cache, state, dtype, pending=None):
        if self.lowerable_with(state):
            # the operations `lower` appends, as a program of their own
            key = (None if cache is None else cache.k.data_ptr(), None if state is None else state.data_ptr())
            alone = self._alone.get(key)
            if alone is None:
                alone = self._alone[key] = OneOp(dtype, h.shape[1], 0,
                                                 lambda program: self.lower(program, cache, state))
            _logits, _x, left = alone.run(step, h, pending=pending)
            return left
        # a sublayer that stays with Python: the same sum, put together here
        x = self.norm.forward(h, dtype, partials=pending)
        y = ops.zeros_like_stream(h)
        left_mixer = self.mixer.forward(x, step, cache, state, y)
        left_ffn = None if self.ffn is None else self.ffn.forward(x, step, y)
        ops.scaled_add(h, y, self.residual_mult, left_mixer, left_ffn)
        return None
