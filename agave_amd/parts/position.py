"""Position encodings applied to queries and keys.

``rope``: rotation of the pairs (i, i + rotary_dim/2), or (2i, 2i + 1) if ``interleaved``, by ``pos/factor * theta^(-2i/rotary_dim)``
(``src/backend/kernels/cpu/rope.zig:11-48``; linear scaling multiplies the position by
``1/factor`` first, ``src/models/gemma3.zig:884-902``).  The frequencies are a table of 32-bit
floats, rounded once from their exact values; the angle and its sine and cosine are computed
in 32-bit inside the q/k kernel.  ``none``: nothing is applied.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import numpy as np
import torch

from ..config.spec import PositionSpec
from .base import BuildEnv, register


class RotaryPosition:
    def __init__(self, spec: PositionSpec, env: BuildEnv):
        if spec.rotary_dim < 2 or spec.rotary_dim % 2:
            raise ValueError(f"rotary_dim must be even and >= 2, got {spec.rotary_dim}")
        if spec.theta <= 0 or spec.factor <= 0:
            raise ValueError("rope needs theta > 0 and factor > 0")
        i = np.arange(spec.rotary_dim // 2, dtype=np.float64)
        inv = np.exp(-np.log(float(spec.theta)) * (2.0 * i) / spec.rotary_dim)
        self.inv_freq = torch.from_numpy(inv.astype(np.float32)).to(env.device)
        self.pos_scale = float(np.float32(1.0) / np.float32(spec.factor))
        self.rotary_dim = spec.rotary_dim
        self.interleaved = bool(spec.interleaved)
        self._exact = inv / float(spec.factor)
        self.magnitude = 1.0           # a factor on sine and cosine (1: a pure rotation)
        self._freq64: Optional[torch.Tensor] = None
        self._device = env.device

    def fused_rotation(self) -> Tuple[Optional[torch.Tensor], float]:
        return self.inv_freq, self.pos_scale

    def rotation_table(self) -> Tuple[Optional[torch.Tensor], bool]:
        """(frequencies as float64, position scaling folded in; whether the pairs are interleaved), for
        kernels that make the angle in double."""
        if self._freq64 is None:
            self._freq64 = torch.from_numpy(self._exact.astype(np.float64)).to(self._device)
        return self._freq64, self.interleaved


class YarnRotaryPosition(RotaryPosition):
    """The same rotation with YaRN's frequencies: pair i's frequency ``f_i = theta^(-2i/d)`` becomes
    ``f_i / s * r_i + f_i (1 - r_i)`` for the factor s, with ``r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1)``,
    ``lo = max(floor(w(fast)), 0)``, ``hi = min(ceil(w(slow)), d - 1)`` and ``w(t) = d ln(original / (2 pi t)) / (2 ln theta)``:
    pairs that turn often within the original context keep their frequency, pairs that turn less than once are slowed
    down by s, those between are blended.  Sine and cosine are multiplied by ``magnitude = slope ln(s) + 1``.  The
    frequencies are made in double; a kernel that makes the angle in double reads them through ``rotation_table``."""

    def __init__(self, spec: PositionSpec, env: BuildEnv):
        super().__init__(PositionSpec("rope", rotary_dim=spec.rotary_dim, theta=spec.theta, interleaved=spec.interleaved), env)
        if spec.yarn_factor <= 0 or spec.yarn_original < 1 or spec.yarn_fast <= 0 or spec.yarn_slow <= 0 or spec.theta == 1.0:
            raise ValueError("rope_yarn needs a positive factor, original context, fast and slow turn counts, and theta != 1")
        d = spec.rotary_dim

        def where(turns: float) -> float:
            return d * math.log(spec.yarn_original / (2.0 * math.pi * turns)) / (2.0 * math.log(spec.theta))
        lo, hi = max(math.floor(where(spec.yarn_fast)), 0), min(math.ceil(where(spec.yarn_slow)), d - 1)
        i = np.arange(d // 2, dtype=np.float64)
        ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
        self._exact = self._exact / float(spec.yarn_factor) * ramp + self._exact * (1.0 - ramp)
        self.inv_freq = torch.from_numpy(self._exact.astype(np.float32)).to(env.device)
        self.magnitude = float(spec.yarn_magnitude_slope * math.log(spec.yarn_factor) + 1.0)

    def fused_rotation(self):
        raise ValueError("rope_yarn scales sine and cosine: the q/k kernel of the plain rotation does not apply it")


class NoPosition:
    def __init__(self, spec: PositionSpec, env: BuildEnv):
        pass

    def fused_rotation(self) -> Tuple[Optional[torch.Tensor], float]:
        return None, 1.0

    def rotation_table(self) -> Tuple[Optional[torch.Tensor], bool]:
        return None, False


register("position", "rope", RotaryPosition)
register("position", "rope_yarn", YarnRotaryPosition)
register("position", "none", NoPosition)
