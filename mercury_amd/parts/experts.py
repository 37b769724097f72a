"""A feed-forward of routed experts."""

from __future__ import annotations

import torch

from ..hostcore import core
from .base import FeedForward, TensorSpec
from .feedforward import ACTIVATION_CODES
from .lowering import OneOp

DEFAULT_NAMES = {"router": "router", "expert": "e{}.", "gate": "gate", "up": "up", "down": "down",
                 "shared": "shared.", "shared_gate": "shared.sg"}


class RoutedExperts(FeedForward):
    """`experts` small gated feed-forwards without biases, of which each token uses `top`.

        s = softmax(W_router x)                 (float32, over all experts)
        E = the `top` experts of largest s      (ties: the lower index)
        w_e = scale * s_e  (s_e / sum_{E} s first, when `renormalize`)
        y = sum_{e in E} w_e * W_down[e] act(W_gate[e] x, W_up[e] x)

    `activation` and its constants are those of :class:`GatedMLP`.  A token's sum runs over
    its experts in the order they were chosen, whatever else is in the batch.
    (With `renormalize` and scale 1 the weights are the softmax over the chosen logits alone.)

    `shared`: a :class:`GatedMLP` every token runs beside its chosen experts, stored under
    ``<shared>``; its output is added to the sum, multiplied, when `shared_gated`, by
    sigmoid(w_sg . x), one number per token (``<shared_gate>.weight`` [1, hidden]).
    """

    graph_safe = True
    lowerable = True

    def __init__(self, hidden: int, experts: int, top: int, intermediate: int,
                 scale: float = 1.0, renormalize: bool = False, activation: str = "silu",
                 limit: float = 0.0, alpha: float = 1.0, beta: float = 0.0,
                 names: dict | None = None, shared=None, shared_gated: bool = False):
        if activation not in ACTIVATION_CODES:
            raise ValueError(f"activation {activation!r} is not implemented; known: {sorted(ACTIVATION_CODES)}")
        self.hidden, self.experts, self.top = int(hidden), int(experts), int(top)
        self.intermediate = int(intermediate)
        if not 0 < self.top <= self.experts:
            raise ValueError(f"top {self.top} of {self.experts} experts")
        self.scale, self.renormalize = float(scale), bool(renormalize)
        self.activation = activation
        self.limit, self.alpha, self.beta = float(limit), float(alpha), float(beta)
        self.names = {**DEFAULT_NAMES, **(names or {})}
        self.shared, self.shared_gated = shared, bool(shared_gated)
        if self.shared is not None and self.shared.hidden != self.hidden:
            raise ValueError("the shared expert reads and writes the model width")
        if self.shared_gated and self.shared is None:
            raise ValueError("a gate without a shared expert")
        self.w_router = self.w_gate_up = self.w_down = self.w_shared_gate = None
        self._alone = None

    def _expert(self, e: int, leaf: str) -> str:
        return f"{self.names['expert'].format(e)}{self.names[leaf]}.weight"

    def param_specs(self) -> dict:
        i, h = self.intermediate, self.hidden
        specs = {f"{self.names['router']}.weight": TensorSpec((self.experts, h))}
        for e in range(self.experts):
            specs[self._expert(e, "gate")] = TensorSpec((i, h))
            specs[self._expert(e, "up")] = TensorSpec((i, h))
            specs[self._expert(e, "down")] = TensorSpec((h, i))
        if self.shared is not None:
            for name, spec in self.shared.param_specs().items():
                specs[self.names["shared"] + name] = spec
            if self.shared_gated:
                specs[f"{self.names['shared_gate']}.weight"] = TensorSpec((1, h))
        return specs

    def bind(self, params, dtype, device) -> None:
        self.w_router = params[f"{self.names['router']}.weight"]
        # [experts, gate rows | up rows, hidden] and [experts, hidden, intermediate]
        self.w_gate_up = torch.stack([
            torch.cat([params[self._expert(e, "gate")], params[self._expert(e, "up")]], dim=0)
            for e in range(self.experts)]).contiguous()
        self.w_down = torch.stack([params[self._expert(e, "down")]
                                   for e in range(self.experts)]).contiguous()
        if self.shared is not None:
            prefix = self.names["shared"]
            gate_name = f"{self.names['shared_gate']}.weight"
            self.shared.bind({n[len(prefix):]: t for n, t in params.items()
                              if n.startswith(prefix) and n != gate_name}, dtype, device)
            if self.shared_gated:
                self.w_shared_gate = params[gate_name].reshape(-1).contiguous()
        self._alone = None

    def weight_bytes(self) -> int:
        """Bytes a step of one token reads: the router and `top` experts."""
        per_expert = 3 * self.intermediate * self.hidden * self.w_down.element_size()
        shared = 0 if self.shared is None else self.shared.weight_bytes()
        return (self.w_router.numel() * self.w_router.element_size() + self.top * per_expert
                + shared)

    def lower(self, program) -> None:
        program.append("routed_experts", core.routed_experts_params(
            w_router=self.w_router.data_ptr(), w_gate_up=self.w_gate_up.data_ptr(),
            w_down=self.w_down.data_ptr(), experts=self.experts, top=self.top,
            ff=self.intermediate, scale=self.scale, renormalize=self.renormalize,
            act=ACTIVATION_CODES[self.activation], limit=self.limit, alpha=self.alpha,
            beta=self.beta, **self._shared_params()))

    def _shared_params(self) -> dict:
        s = self.shared
        if s is None:
            return {}
        return dict(shared_gate_up=s.w_gate_up.data_ptr(), shared_down=s.w_down.data_ptr(),
                    shared_gate=0 if self.w_shared_gate is None else self.w_shared_gate.data_ptr(),
                    shared_ff=s.intermediate, shared_act=ACTIVATION_CODES[s.activation],
                    shared_limit=s.limit, shared_alpha=s.alpha, shared_beta=s.beta)

    def forward(self, x, step, accum):
        if self._alone is None:
            self._alone = OneOp(x.dtype, self.hidden, 0, self.lower)
        _logits, _x, pending = self._alone.run(step, accum, x=x)
        return pending
