"""Rotary position embedding as a part.

Half-split pairing as the reference computes it (src/kernels/rope.cu:28-60): for i in
[0, rot/2): angle = pos / theta^(2i/rot); (x[i], x[i + rot/2]) is rotated by that angle.
theta is the literal 1e6 in the reference (src/qwen.cc:636) and a parameter here.  The
angles' cosines and sines are tabulated once per position (computed in float64, stored as
float32) and the kernel looks them up; the table grows when a longer position shows up.

Two things are parameters beyond the reference: which entries form a pair (``pairing``:
"half", entry i with entry i + rot/2, or "interleaved", entry 2i with entry 2i + 1; the table is
the same, the kernels that rotate differ) and a stretching of the frequencies for contexts
longer than the one trained on (``scaling``, the YaRN rule: with dim(t) = rot ln(original /
(2 pi t)) / (2 ln theta), lo = max(floor(dim(fast)), 0), hi = min(ceil(dim(slow)), rot - 1) and
ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), frequency i becomes f_i / factor * ramp_i +
f_i (1 - ramp_i), and cosines and sines are multiplied by 0.1 ln(factor) + 1).  A ``scaling`` with
``kind`` "wavelength" goes by each frequency's wavelength l = 2 pi / f against the ``original`` context:
f is kept where l < original / high, divided by ``factor`` where l > original / low, and between the two,
with s = (original / l - low) / (high - low), it becomes (1 - s) f / factor + s f; nothing else changes.
"""
from __future__ import annotations

import math
from typing import Any, Dict, Optional

import torch

from ..config.registry import POSITION_ENCODINGS
from .base import BuildContext, Part


class _SharedTable:
    """One table for all parts of a model with the same rotated size and base (its layers,
    usually), kept in the model's ``BuildContext.shared``: ``generation`` counts how often it
    has been made anew."""

    def __init__(self) -> None:
        self.table: Optional[torch.Tensor] = None
        self.generation = 0


@POSITION_ENCODINGS.register("rotary")
class Rotary(Part):
    def __init__(self, rotary_dim: int, theta: float, max_positions: int = 0, pairing: str = "half",
                 scaling: Optional[Dict[str, Any]] = None):
        super().__init__(rotary_dim=rotary_dim, theta=theta, max_positions=max_positions,
                         pairing=pairing, scaling=scaling)
        if rotary_dim % 2:
            raise ValueError(f"rotary: the rotated size {rotary_dim} must be even")
        if pairing not in ("half", "interleaved"):
            raise ValueError(f"rotary: pairing '{pairing}' is neither 'half' nor 'interleaved'")
        self.rotary_dim, self.theta, self.pairing = int(rotary_dim), float(theta), pairing
        self.scaling = None
        self.scaling_kind = str(scaling.get("kind", "yarn")) if scaling else None
        if scaling and self.scaling_kind == "wavelength":
            self.scaling = ("wavelength",) + tuple(float(scaling[k]) for k in ("factor", "original", "low", "high"))
            if self.scaling[1] <= 0 or self.scaling[2] <= 0 or self.scaling[4] <= self.scaling[3]:
                raise ValueError("rotary: wavelength scaling needs factor > 0, original > 0 and high > low")
        elif scaling and self.scaling_kind == "yarn":
            self.scaling = tuple(float(scaling[k]) for k in ("factor", "original", "fast", "slow"))
        elif scaling:
            raise ValueError(f"rotary: scaling kind '{self.scaling_kind}' is neither 'yarn' nor 'wavelength'")
        self.initial = int(max_positions)
        self._shared = _SharedTable()
        self._device = None

    def bind(self, tensors, ctx: BuildContext) -> None:
        self._device = ctx.device
        self._shared = ctx.shared.setdefault(("rotary table", self.rotary_dim, self.theta, self.scaling),
                                             _SharedTable())

    def tables_epoch(self) -> int:
        return self._shared.generation

    def ready(self, position: int) -> bool:
        return self.capacity() > position

    @property
    def _table(self) -> Optional[torch.Tensor]:
        return self._shared.table

    def _make(self, count: int) -> torch.Tensor:
        half = self.rotary_dim // 2
        i = torch.arange(half, dtype=torch.float64)
        inv_freq = 1.0 / torch.pow(torch.tensor(self.theta, dtype=torch.float64),
                                   2.0 * i / self.rotary_dim)
        magnitude = 1.0
        if self.scaling is not None and self.scaling[0] == "wavelength":
            _, factor, original, low, high = self.scaling
            wavelength = 2.0 * math.pi / inv_freq
            blend = (original / wavelength - low) / (high - low)
            between = (1.0 - blend) * inv_freq / factor + blend * inv_freq
            inv_freq = torch.where(wavelength < original / high, inv_freq,
                                   torch.where(wavelength > original / low, inv_freq / factor, between))
        elif self.scaling is not None:
            factor, original, fast, slow = self.scaling

            def turn_dim(turns: float) -> float:
                return self.rotary_dim * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(self.theta))

            lo = max(math.floor(turn_dim(fast)), 0)
            hi = min(math.ceil(turn_dim(slow)), self.rotary_dim - 1)
            ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
            inv_freq = inv_freq / factor * ramp + inv_freq * (1.0 - ramp)
            magnitude = 0.1 * math.log(factor) + 1.0
        angle = torch.arange(count, dtype=torch.float64)[:, None] * inv_freq[None, :]
        table = (torch.cat([torch.cos(angle), torch.sin(angle)], dim=1) * magnitude).to(torch.float32)
        return table.contiguous().to(self._device)

    def rotary_table(self, max_position: int) -> torch.Tensor:
        """float32 [positions, rot]: cosines in the first half of a row, sines in the second."""
        need = max_position + 1
        if self._table is None or self._table.shape[0] < need:
            count = max(need, min(self.initial, 16384), 256)
            if self._table is not None:
                count = max(count, 2 * self._table.shape[0])
            self._shared.table = self._make(count)
            self._shared.generation += 1
        return self._table

    def capacity(self) -> int:
        """Positions the present table covers."""
        return 0 if self._table is None else int(self._table.shape[0])

    def apply(self, qkv, nh, nkv, d, positions) -> None:  # the table path covers this part
        raise NotImplementedError
