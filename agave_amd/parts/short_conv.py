"""A short causal convolution over time on every channel, with its state.

``y[t, c] = act(b[c] + sum_j w[c, j] * u[t - taps + 1 + j, c])`` (the bias ``b`` is optional): the last column of ``w`` multiplies the
current token's input, and inputs before the sequence's start are zeros.  The last ``taps - 1``
inputs of every sequence are kept as state, so that a sequence fed in pieces, or token by token,
sees what a whole pass would.  Several tensors that are convolved alike (the q, k and v of one
mixer) are stacked along the channels and run as one kernel.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from ..cache import StateNeed
from ..ops import sequence as seq_ops
from .base import BuildEnv


class ShortConv:
    def __init__(self, weights: Sequence[torch.Tensor], env: BuildEnv, silu: bool, name: str = "conv",
                 bias: Optional[torch.Tensor] = None):
        taps = {int(w.shape[1]) for w in weights}
        if len(taps) != 1:
            raise ValueError(f"{name}: stacked convolutions must have the same number of taps, got {sorted(taps)}")
        self.taps = taps.pop()
        if not 1 <= self.taps <= seq_ops.MAX_TAPS:
            raise ValueError(f"{name}: {self.taps} taps (1 to {seq_ops.MAX_TAPS} are supported)")
        self.weight = torch.cat([w.to(torch.float32) for w in weights], dim=0).contiguous().to(env.device)
        self.channels = self.weight.shape[0]
        self.silu = bool(silu)
        self.env = env
        self.bias = None
        if bias is not None:
            if tuple(bias.shape) != (self.channels,):
                raise ValueError(f"{name}: a bias of shape {tuple(bias.shape)} for {self.channels} channels")
            self.bias = bias.to(torch.float32).contiguous().to(env.device)

    def state_need(self) -> StateNeed:
        return StateNeed((self.taps - 1, self.channels), torch.float32)

    def forward(self, u: torch.Tensor, out: torch.Tensor, state: torch.Tensor, step, in_bias: Optional[torch.Tensor] = None) -> None:
        """``u`` and ``out``: float32 [N, channels] (column slices are fine); ``state`` is advanced.  ``in_bias``
        [channels] float32 is added to the inputs on the way in."""
        seq_ops.short_conv(u, self.weight, out, state, step, self.silu, self.bias, in_bias)
