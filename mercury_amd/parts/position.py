"""Position encodings applied to queries and keys inside a mixer."""

from __future__ import annotations

import math

import torch

from .base import PositionDescriptor, PositionEncoding


class RotaryPosition(PositionEncoding):
    """Rotary encoding: dims j and j + rotary_dim/2 of a head (the half-split layout; with
    `interleaved`, dims 2j and 2j + 1) form a pair that is turned by the angle
    position * theta^(-2j/rotary_dim).

    The angle table is built as the reference builds it (mercury/model/rope.py:37-47):
    inverse frequencies, positions and their outer product in float32, then cos and sin.
    The reference then casts the table to the model dtype; here it stays float32 and the
    rotation is computed in float32, whatever the activations' dtype.  Positions are absolute
    within the sequence, so keys can be cached after rotation.
    """

    def __init__(self, head_dim: int, theta: float, rotary_dim: int | None = None,
                 interleaved: bool = False, scaling: tuple | None = None):
        self.head_dim = int(head_dim)
        self.theta = float(theta)
        self.interleaved = bool(interleaved)
        self.rotary_dim = int(head_dim if rotary_dim is None else rotary_dim)
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError(f"rotary width {self.rotary_dim} must be even and within the head")
        # (factor, low, high, original): frequencies slowed where the wavelength is long
        self.scaling = tuple(float(v) for v in scaling) if scaling else None
        if self.scaling:
            factor, low, high, original = self.scaling
            if not (factor > 0 and high > low >= 0 and original > 0):
                raise ValueError("frequency scaling: factor > 0, high > low >= 0, original > 0")
        self.cos = None
        self.sin = None

    def frequencies(self) -> torch.Tensor:
        """Angle per position step of every pair, float64.  With `scaling`, a pair whose
        wavelength 2 pi / f is below original / high keeps f, one above original / low turns
        at f / factor, and between the two f / factor and f are blended linearly in
        original / wavelength."""
        exponents = torch.arange(0, self.rotary_dim, 2, dtype=torch.float64) / self.rotary_dim
        f = self.theta ** -exponents
        if not self.scaling:
            return f
        factor, low, high, original = self.scaling
        turns = original * f / (2.0 * math.pi)        # original / wavelength
        blend = ((turns - low) / (high - low)).clamp(0.0, 1.0)
        mixed = (1.0 - blend) * f / factor + blend * f
        return torch.where(turns > high, f, torch.where(turns < low, f / factor, mixed))

    def prepare(self, max_positions: int, device) -> None:
        if self.cos is not None and self.cos.shape[0] >= max_positions \
                and self.cos.device == torch.device(device):
            return  # a part shared by several layers is prepared once
        if self.scaling:
            # position * frequency in float64, so that the table is the angle's own cos and sin
            angles = torch.outer(torch.arange(max_positions, dtype=torch.float64), self.frequencies())
        else:
            exponents = torch.arange(0, self.rotary_dim, 2, dtype=torch.float32) / self.rotary_dim
            inv_freq = 1.0 / (self.theta ** exponents)
            positions = torch.arange(max_positions, dtype=torch.float32)
            angles = torch.outer(positions, inv_freq)
        self.cos = angles.cos().float().contiguous().to(device)
        self.sin = angles.sin().float().contiguous().to(device)

    def describe(self) -> PositionDescriptor:
        return PositionDescriptor(self.rotary_dim, self.cos, self.sin, self.interleaved)


class NoPosition(PositionEncoding):
    """Queries and keys are used as projected."""

    def describe(self) -> PositionDescriptor:
        return PositionDescriptor()
