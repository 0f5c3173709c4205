"""A gated linear recurrence per channel beside a GELU branch, as a mixer (the recurrent block of Griffin:
De, Smith, Fernando et al., "Griffin: Mixing Gated Linear Recurrences with Local Attention for Efficient Language Models").

In the order of its steps: both branches' products in one (``[y | x]``, with their biases, 32-bit rows); a short causal
convolution with a bias on the x branch; in every block of channels the two gates' products and sigmoids, the decay
``a = exp(-c r softplus(lam))`` and the gated input ``sqrt(1 - a^2) g u``; the recurrence ``S <- a S + input`` along
each sequence; ``S gelu_tanh(y)``; the output product.  Between the first product and the rows of the output product
everything is 32-bit.  State per sequence: S [width] and the convolution's last ``taps - 1`` inputs.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..cache import GroupKey, StateNeed
from ..config.spec import RglruSpec
from ..ops import rglru as ops
from ..weights.loader import TensorNeed
from .base import BuildEnv, register, state_tensor
from .linear import Linear
from .short_conv import ShortConv


class Rglru:
    @staticmethod
    def kernel_libraries(spec, dtype):
        return ("rglru", "sequence")

    def __init__(self, spec: RglruSpec, weights, env: BuildEnv):
        s = spec
        if s.blocks < 1 or s.width % s.blocks:
            raise ValueError(f"rglru: {s.width} channels do not form {s.blocks} equal blocks")
        self.spec, self.env = spec, env
        # (the branches' biases are added where their rows are read next: by the convolution and by the scan's read-out)
        self.proj = Linear([weights.get(s.y_proj), weights.get(s.x_proj)], env, "rglru_in")

        def bias(name):
            return weights.get(name).to(torch.float32).reshape(-1).contiguous().to(env.device) if name else None
        self.y_bias, self.x_bias = bias(s.y_bias), bias(s.x_bias)
        self.conv = ShortConv([weights.get(s.conv)], env, silu=False, name="rglru_conv",
                              bias=weights.get(s.conv_bias) if s.conv_bias else None)
        if self.conv.channels != s.width:
            raise ValueError(f"rglru: the convolution has {self.conv.channels} channels, the branch {s.width}")
        gate_dtype = env.weight_dtype(weights.get(s.r_gate).dtype)
        self.w_r = weights.get(s.r_gate).to(gate_dtype).contiguous().to(env.device)
        self.w_i = weights.get(s.i_gate).to(gate_dtype).contiguous().to(env.device)

        def vec(name):
            return weights.get(name).to(torch.float32).reshape(-1).contiguous().to(env.device)
        self.b_r, self.b_i = vec(s.r_bias), vec(s.i_bias)
        # decay_scale * softplus(lam), once, in double
        lam = weights.get(s.lam).to(torch.float64).reshape(-1)
        self.decay = (float(s.decay_scale) * torch.nn.functional.softplus(lam)).to(torch.float32).contiguous().to(env.device)
        self.o = Linear([weights.get(s.o_proj)], env, "rglru_o")

    @staticmethod
    def tensor_needs(spec: RglruSpec) -> List[TensorNeed]:
        s = spec
        bw = s.width // max(s.blocks, 1)
        needs = [TensorNeed(s.y_proj, (s.width, s.hidden)), TensorNeed(s.x_proj, (s.width, s.hidden)),
                 TensorNeed(s.conv, (s.width, s.conv_taps))]
        for name in (s.y_bias, s.x_bias, s.conv_bias):
            if name:
                needs.append(TensorNeed(name, (s.width,)))
        needs += [TensorNeed(s.r_gate, (s.blocks, bw, bw)), TensorNeed(s.r_bias, (s.blocks, bw)),
                  TensorNeed(s.i_gate, (s.blocks, bw, bw)), TensorNeed(s.i_bias, (s.blocks, bw)),
                  TensorNeed(s.lam, (s.width,)), TensorNeed(s.o_proj, (s.hidden, s.width))]
        return needs

    def kv_need(self) -> Optional[GroupKey]:
        return None

    def state_need(self) -> Dict[str, StateNeed]:
        return {"S": StateNeed((self.spec.width,), torch.float32), "conv": self.conv.state_need()}

    def forward(self, x: torch.Tensor, step, memory: int, writes: bool = True) -> torch.Tensor:
        s, ws = self.spec, self.env.workspace
        n, w = x.shape[0], s.width
        if not writes:
            raise ValueError("a recurrent mixer advances its own state; it cannot read another run's")
        proj = self.proj.forward(x, out_dtype=torch.float32, tag="rglru_in")
        y, xb = ws.columns(proj, (0, w, 2 * w))
        u = ws.get("rglru_conved", n, w, torch.float32)
        self.conv.forward(xb, u, state_tensor(step, memory, "conv"), step, in_bias=self.x_bias)
        a = ws.get("rglru_decay", n, w, torch.float32)
        gx = ws.get("rglru_input", n, w, torch.float32)
        ops.gates(u, self.w_r, self.w_i, self.b_r, self.b_i, self.decay, a, gx)
        ctx = ws.get("rglru_ctx", n, w, self.env.dtype)
        ops.scan(a, gx, y, ctx, state_tensor(step, memory, "S"), step, ws, y_bias=self.y_bias)
        return self.o.forward(ctx, tag="rglru_o", slices_ok=True)


register("mixer", "rglru", Rglru)
