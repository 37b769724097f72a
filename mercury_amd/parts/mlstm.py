"""A matrix memory with an input gate, a forget gate and a running maximum (the mLSTM cell),
carried as per-request state."""

from __future__ import annotations

import torch

from ..hostcore import core
from ..kernels import ops
from .base import Mixer, StateSpec, TensorSpec
from .lowering import OneOp

DEFAULT_NAMES = {"q": "q_proj", "k": "k_proj", "v": "v_proj", "gate": "g_proj", "o": "o_proj",
                 "input": "i_proj", "forget": "f_proj", "norm": "norm"}


class MatrixMemory(Mixer):
    """Per head h, with q and k of `dim` and v of `vdim` columns (no biases) and one input and
    one forget gate a head (biased):

        q_t = (W_q x)_h * q_scale                    (default dim^-1/2)
        i_t = cap tanh((w_i . x + b_i) / cap),  f_t = logsigmoid(cap tanh((w_f . x + b_f) / cap))
        m_t = max(f_t + m_(t-1), i_t)
        S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T
        n_t = exp(f_t + m_(t-1) - m_t) n_(t-1) + exp(i_t - m_t) k_t
        o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)

    S, n and m are zero before the sequence (m starts at zero).  `gate_cap` None or 0: the
    gates' logits are not bounded.  Each head's o is divided by its root mean square over vdim
    (eps inside the root); the heads side by side are multiplied by a weight over all their
    columns and by sigmoid(W_g x), and projected by W_o.  Everything between the input
    projection and the output projection is float32; S, n and m of every head are the state a
    request carries from step to step, one float32 row per request slot (zeroed when a
    request takes the slot).
    """

    graph_safe = True
    lowers_state = True
    lowerable = True

    def __init__(self, hidden: int, heads: int, dim: int, vdim: int, gate_cap: float | None = None,
                 eps: float = 1e-6, q_scale: float | None = None, names: dict | None = None):
        self.hidden, self.heads, self.dim, self.vdim = int(hidden), int(heads), int(dim), int(vdim)
        if min(self.hidden, self.heads, self.dim, self.vdim) <= 0:
            raise ValueError("a matrix memory's sizes are positive")
        self.gate_cap = float(gate_cap) if gate_cap else 0.0
        if self.gate_cap < 0:
            raise ValueError("the bound on the gates' logits is positive, or absent")
        self.eps = float(eps)
        self.q_scale = float(q_scale) if q_scale is not None else self.dim ** -0.5
        self.names = {**DEFAULT_NAMES, **(names or {})}
        self.w_in = self.b_in = self.w_out = self.norm = None
        self._alone: dict = {}

    def state_floats(self) -> int:
        """Floats of state per request, as the recurrence kernel lays it out (what
        ``core.mlstm_state_floats`` answers once the kernel library is loaded): S of every
        head, then n and m once for each of a head's workgroups of 28 columns."""
        if self.dim > 256:
            raise ValueError("the recurrence kernel holds memories of up to 256 rows")
        copies = -(-self.vdim // 28)
        return self.heads * (self.dim * self.vdim + copies * (self.dim + 1))

    def state_spec(self) -> StateSpec:
        return StateSpec((self.state_floats(),), torch.float32)

    def param_specs(self) -> dict:
        n, h = self.names, self.hidden
        qk, inner = self.heads * self.dim, self.heads * self.vdim
        return {
            f"{n['q']}.weight": TensorSpec((qk, h)),
            f"{n['k']}.weight": TensorSpec((qk, h)),
            f"{n['v']}.weight": TensorSpec((inner, h)),
            f"{n['gate']}.weight": TensorSpec((inner, h)),
            f"{n['input']}.weight": TensorSpec((self.heads, h)),
            f"{n['input']}.bias": TensorSpec((self.heads,), role="vector"),
            f"{n['forget']}.weight": TensorSpec((self.heads, h)),
            f"{n['forget']}.bias": TensorSpec((self.heads,), role="vector"),
            f"{n['norm']}.weight": TensorSpec((inner,), role="vector", init="one_plus_normal"),
            f"{n['o']}.weight": TensorSpec((h, inner)),
        }

    def bind(self, params, dtype, device) -> None:
        n = self.names
        # one projection for all six: rows [q | k | v | gate | input gate | forget gate]
        keys = ("q", "k", "v", "gate", "input", "forget")
        self.w_in = torch.cat([params[f"{n[key]}.weight"] for key in keys], dim=0).contiguous()
        quiet = self.w_in.shape[0] - 2 * self.heads
        self.b_in = torch.cat([
            torch.zeros(quiet, dtype=torch.float32, device=self.w_in.device),
            params[f"{n['input']}.bias"].float(), params[f"{n['forget']}.bias"].float()]).contiguous()
        self.w_out = params[f"{n['o']}.weight"]
        self.norm = params[f"{n['norm']}.weight"].float().contiguous()
        self._alone.clear()

    def weight_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.w_in, self.b_in, self.w_out, self.norm))

    def lower(self, program, cache=None, state=None) -> None:
        if state is None:
            raise ValueError("a matrix memory runs over a state tensor")
        if state.dtype != torch.float32 or state.dim() != 2:
            raise ValueError("the state is float32 [slots, floats]")
        program.append("mlstm", core.mlstm_params(
            w_in=self.w_in.data_ptr(), b_in=self.b_in.data_ptr(), b_in_dtype=ops.F32,
            w_out=self.w_out.data_ptr(), norm=self.norm.data_ptr(), heads=self.heads,
            dim=self.dim, vdim=self.vdim, q_scale=self.q_scale, gate_cap=self.gate_cap,
            eps=self.eps, state=state.data_ptr(), slot_floats=state.shape[1]))

    def forward(self, x, step, cache, state, accum):
        alone = self._alone.get(state.data_ptr())
        if alone is None:
            alone = self._alone[state.data_ptr()] = OneOp(
                x.dtype, self.hidden, 0, lambda program: self.lower(program, None, state))
        _logits, _x, pending = alone.run(step, accum, x=x)
        return pending
