"""Feed-forward parts."""

from __future__ import annotations

import torch

from ..hostcore import core
from .base import FeedForward, TensorSpec
from .lowering import OneOp

ACTIVATIONS = ("silu", "swish_clamp", "gelu_tanh")
# the kernels' codes of the activations
ACTIVATION_CODES = {"silu": 0, "swish_clamp": 1, "gelu_tanh": 2}
DEFAULT_NAMES = {"gate": "gate_proj", "up": "up_proj", "down": "down_proj"}


class GatedMLP(FeedForward):
    """down(act(gate(x), up(x))) without biases.  `activation`:

    ``"silu"``: silu(g) * u (reference: mercury/model/qwen2.py:34-42).
    ``"swish_clamp"``: g' * sigmoid(alpha * g') * (u' + beta) with g' = min(g, limit) and
    u' = clamp(u, -limit, limit).
    ``"gelu_tanh"``: 0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3))) * u.

    `names` maps gate, up, down to the stored tensors' leaf names (default ``gate_proj``,
    ``up_proj``, ``down_proj``)."""

    graph_safe = True
    lowerable = True

    def __init__(self, hidden: int, intermediate: int, activation: str = "silu",
                 names: dict | None = None, limit: float = 0.0, alpha: float = 1.0,
                 beta: float = 0.0):
        if activation not in ACTIVATIONS:
            raise ValueError(f"activation {activation!r} is not implemented; known: {ACTIVATIONS}")
        self.hidden, self.intermediate = int(hidden), int(intermediate)
        self.activation = activation
        self.limit, self.alpha, self.beta = float(limit), float(alpha), float(beta)
        if activation == "swish_clamp" and not self.limit > 0:
            raise ValueError("swish_clamp needs a positive limit")
        self.names = {**DEFAULT_NAMES, **(names or {})}
        self.w_gate_up = self.w_down = None
        self._alone = None

    def param_specs(self) -> dict:
        i, h, n = self.intermediate, self.hidden, self.names
        return {
            f"{n['gate']}.weight": TensorSpec((i, h)),
            f"{n['up']}.weight": TensorSpec((i, h)),
            f"{n['down']}.weight": TensorSpec((h, i)),
        }

    def bind(self, params, dtype, device) -> None:
        n = self.names
        # One projection for gate and up: rows [gate | up].
        self.w_gate_up = torch.cat(
            [params[f"{n['gate']}.weight"], params[f"{n['up']}.weight"]], dim=0
        ).contiguous()
        self.w_down = params[f"{n['down']}.weight"]
        self._alone = None

    def weight_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.w_gate_up, self.w_down))

    def lower(self, program) -> None:
        program.append("gated_mlp", core.gated_mlp_params(
            self.w_gate_up.data_ptr(), self.w_down.data_ptr(), self.intermediate,
            act=ACTIVATION_CODES[self.activation], limit=self.limit, alpha=self.alpha,
            beta=self.beta))

    def forward(self, x, step, accum):
        # the operations `lower` appends, as a program of their own
        if self._alone is None:
            self._alone = OneOp(x.dtype, self.hidden, 0, self.lower)
        _logits, _x, pending = self._alone.run(step, accum, x=x)
        return pending


UNARY_ACTIVATIONS = {"relu2": 0, "gelu_tanh": 1}     # the kernels' codes
UNARY_NAMES = {"up": "up_proj", "down": "down_proj"}


class UnaryMLP(FeedForward):
    """down(act(up(x))) without biases, for an activation of one operand.  `activation`:

    ``"relu2"``: the square of relu.
    ``"gelu_tanh"``: 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3))).

    `names` maps up, down to the stored tensors' leaf names (default ``up_proj``,
    ``down_proj``)."""

    graph_safe = True
    lowerable = True

    def __init__(self, hidden: int, intermediate: int, activation: str = "relu2",
                 names: dict | None = None):
        if activation not in UNARY_ACTIVATIONS:
            raise ValueError(f"activation {activation!r} is not implemented; known: "
                             f"{sorted(UNARY_ACTIVATIONS)}")
        self.hidden, self.intermediate = int(hidden), int(intermediate)
        self.activation = activation
        self.names = {**UNARY_NAMES, **(names or {})}
        self.w_up = self.w_down = None
        self._alone = None

    def param_specs(self) -> dict:
        i, h, n = self.intermediate, self.hidden, self.names
        return {f"{n['up']}.weight": TensorSpec((i, h)), f"{n['down']}.weight": TensorSpec((h, i))}

    def bind(self, params, dtype, device) -> None:
        n = self.names
        self.w_up = params[f"{n['up']}.weight"]
        self.w_down = params[f"{n['down']}.weight"]
        self._alone = None

    def weight_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.w_up, self.w_down))

    def lower(self, program) -> None:
        program.append("unary_mlp", core.unary_mlp_params(
            self.w_up.data_ptr(), self.w_down.data_ptr(), self.intermediate,
            act=UNARY_ACTIVATIONS[self.activation]))

    def forward(self, x, step, accum):
        if self._alone is None:
            self._alone = OneOp(x.dtype, self.hidden, 0, self.lower)
        _logits, _x, pending = self._alone.run(step, accum, x=x)
        return pending
