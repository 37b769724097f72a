"""Retention: linear attention with a fixed decay per head, carried as per-request state."""

from __future__ import annotations

import torch

from ..hostcore import core
from .base import Mixer, PositionEncoding, StateSpec, TensorSpec
from .lowering import OneOp

DEFAULT_NAMES = {"q": "q_proj", "k": "k_proj", "v": "v_proj", "gate": "g_proj", "o": "o_proj"}


class Retention(Mixer):
    """Per head h, with q and k of `dim` and v of `vdim` columns (no biases):

        q_t, k_t  turned by the position encoding (their first dims, by the token's position)
        k_t  <-  k_t * k_scale                       (default dim^-1/2), after the turn
        S_t  =  decay_h S_(t-1) + k_t v_t^T          (S is dim x vdim, zero before the sequence)
        o_t  =  S_t^T q_t

    There is no softmax and no denominator.  Each head's o is divided by its root mean square
    over vdim (eps inside the root, no weight), the heads side by side are multiplied by
    silu(W_g x) and projected by W_o.  Everything between the input projection and the output
    projection is float32; the state a request carries from step to step is S of every head,
    one float32 row per request slot (zeroed when a request takes the slot).
    """

    graph_safe = True
    lowers_state = True

    def __init__(self, hidden: int, heads: int, dim: int, vdim: int, decay,
                 position: PositionEncoding, eps: float = 1e-6, k_scale: float | None = None,
                 names: dict | None = None):
        self.hidden, self.heads, self.dim, self.vdim = int(hidden), int(heads), int(dim), int(vdim)
        if min(self.hidden, self.heads, self.dim, self.vdim) <= 0:
            raise ValueError("a retention mixer's sizes are positive")
        self.decay_values = tuple(float(g) for g in decay)
        if len(self.decay_values) != self.heads:
            raise ValueError(f"{len(self.decay_values)} decays for {self.heads} heads")
        if any(not 0.0 <= g <= 1.0 for g in self.decay_values):
            raise ValueError("a head's decay lies in [0, 1]")
        self.position = position
        self.eps = float(eps)
        self.k_scale = float(k_scale) if k_scale is not None else self.dim ** -0.5
        self.names = {**DEFAULT_NAMES, **(names or {})}
        self.w_in = self.w_out = self.decay = None
        self._alone: dict = {}

    @property
    def lowerable(self) -> bool:
        pos = self.position.describe()
        return pos is not None and not pos.interleaved and pos.distance_slopes is None

    def state_spec(self) -> StateSpec:
        return StateSpec((self.heads * self.dim * self.vdim,), torch.float32)

    def prepare(self, max_positions: int, device) -> None:
        self.position.prepare(max_positions, device)

    def param_specs(self) -> dict:
        n, h = self.names, self.hidden
        qk, inner = self.heads * self.dim, self.heads * self.vdim
        return {
            f"{n['q']}.weight": TensorSpec((qk, h)),
            f"{n['k']}.weight": TensorSpec((qk, h)),
            f"{n['v']}.weight": TensorSpec((inner, h)),
            f"{n['gate']}.weight": TensorSpec((inner, h)),
            f"{n['o']}.weight": TensorSpec((h, inner)),
        }

    def bind(self, params, dtype, device) -> None:
        n = self.names
        # one projection for all four: rows [q | k | v | gate]
        self.w_in = torch.cat([params[f"{n[key]}.weight"] for key in ("q", "k", "v", "gate")],
                              dim=0).contiguous()
        self.w_out = params[f"{n['o']}.weight"]
        self.decay = torch.tensor(self.decay_values, dtype=torch.float32, device=self.w_in.device)
        self._alone.clear()

    def weight_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.w_in, self.w_out))

    def lower(self, program, cache=None, state=None) -> None:
        if state is None:
            raise ValueError("a retention mixer runs over a state tensor")
        if state.dtype != torch.float32 or state.dim() != 2:
            raise ValueError("the state is float32 [slots, floats]")
        pos = self.position.describe()
        if pos is None or pos.interleaved or pos.distance_slopes is not None:
            raise ValueError("retention turns q and k by tabulated angles in the half-split layout")
        ptr = lambda t: 0 if t is None else t.data_ptr()
        program.append("retention", core.retention_params(
            w_in=self.w_in.data_ptr(), w_out=self.w_out.data_ptr(), decay=self.decay.data_ptr(),
            heads=self.heads, dim=self.dim, vdim=self.vdim, k_scale=self.k_scale, eps=self.eps,
            rotary_dim=pos.rotary_dim, cos=ptr(pos.cos), sin=ptr(pos.sin),
            table_positions=0 if pos.cos is None else pos.cos.shape[0],
            state=state.data_ptr(), slot_floats=state.shape[1]))

    def forward(self, x, step, cache, state, accum):
        alone = self._alone.get(state.data_ptr())
        if alone is None:
            alone = self._alone[state.data_ptr()] = OneOp(
                x.dtype, self.hidden, 0, lambda program: self.lower(program, None, state))
        _logits, _x, pending = alone.run(step, accum, x=x)
        return pending
