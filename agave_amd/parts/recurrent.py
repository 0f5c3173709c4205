"""Mixers with a matrix of state per head that is advanced token by token.

Both keep ``S`` [head_dim, v_head_dim] per sequence and head in 32-bit (stored with a column's rows
together, ``[heads, v_head_dim, head_dim]``) and compute, for every token,

    S <- diag(a) S;   S <- S + k u^T;   o = S^T q          (the read-out sees the token's own write)

``gated_delta`` (a delta rule with a decay per head and key channel): q, k and v pass a short causal
convolution and SiLU; q and k become unit vectors per head (q also times head_dim^-1/2); head h reads
the q/k head ``h // (n_heads / n_kv_heads)``; ``a = exp(-exp(decay_log_h) * softplus(W_out (W_in x) + bias))``;
``u = sigmoid(W_beta x)_h * (v - S^T k)`` with the decayed S.  The read-out is divided by its root mean
square per head, times a gain shared by the heads, times ``sigmoid(W_gate_out (W_gate_in x))``.

``hgrn2`` (linear attention whose forget gate also sets what is written): ``q = silu(W_q x)``,
``f = lower + (1 - lower) * sigmoid(W_f x + b_f)``, ``a = f``, ``k = 1 - f``, ``u = v = W_v x``; the
read-out gets an RMS norm per head with a gain shared by the heads.

``mamba2`` (a state-space mixer with one decay per head and token): one product gives ``[z | xs | B | C | dt]``;
``xs``, ``B`` and ``C`` pass one short causal convolution with a bias and SiLU; ``d = softplus(dt + dt_bias)``;
``a = exp(-exp(A_log_h) d)`` for every key channel, ``k = B`` and ``q = C`` of the head's group, ``u = d xs``; the
read-out gets ``D_h xs`` on top, is multiplied by ``silu(z)``, divided by its root mean square in equal parts of the
row, and multiplied by a weight.

The gates, decays, unit vectors and the state are 32-bit whatever the engine's element type; the
first products write 32-bit rows for that reason.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..cache import GroupKey, StateNeed
from ..config.spec import GatedDeltaSpec, Hgrn2Spec, Mamba2Spec
from ..ops import sequence as seq_ops
from ..weights.loader import TensorNeed
from .base import BuildEnv, register, state_tensor
from .linear import Linear
from .short_conv import ShortConv


def _vec(weights, name: str, env: BuildEnv) -> torch.Tensor:
    return weights.get(name).to(torch.float32).contiguous().view(-1).to(env.device)


class GatedDelta:
    @staticmethod
    def kernel_libraries(spec, dtype):
        return ("sequence",)

    def __init__(self, spec: GatedDeltaSpec, weights, env: BuildEnv, own_output: bool = True, own_input: bool = True):
        s = spec
        if s.n_heads % s.n_kv_heads:
            raise ValueError("heads must be a multiple of the query/key heads")
        self.spec, self.env = spec, env
        self.state_prefix = ""
        self.kd, self.vd, self.hd = s.n_kv_heads * s.head_dim, s.n_heads * s.v_head_dim, s.n_heads * s.head_dim
        self.context_width = self.vd
        a1, g1 = weights.get(s.decay_in), weights.get(s.gate_in)
        # q, k, v, the write strength's logit and the inner rows of the decay and of the gate: one product
        mats = [weights.get(s.q_proj), weights.get(s.k_proj), weights.get(s.v_proj), weights.get(s.beta_proj), a1, g1]
        self.input_matrices = None if own_input else mats
        self.input_width = sum(int(m.shape[0]) for m in mats)
        self.proj = Linear(mats, env, "delta_in") if own_input else None
        self.ra, self.rg = int(a1.shape[0]), int(g1.shape[0])
        # the second steps read 32-bit rows, so they run on the plain product whatever the engine's type
        self.decay_out = Linear([weights.get(s.decay_out)], env, "delta_decay", pack=False)
        self.gate_out = Linear([weights.get(s.gate_out)], env, "delta_gate", pack=False)
        self.conv = (ShortConv([weights.get(s.q_conv), weights.get(s.k_conv), weights.get(s.v_conv)], env, silu=True,
                               name="delta_conv") if s.conv_taps else None)
        if self.conv is None:
            raise ValueError("gated delta rule: the convolution with its SiLU is part of the mixer (conv_taps >= 1)")
        self.a_log = _vec(weights, s.decay_log, env)
        self.dt_bias = _vec(weights, s.decay_bias, env)
        self.norm_gain = _vec(weights, s.out_norm, env)
        self.o_weight = weights.get(s.o_proj)
        self.o = Linear([self.o_weight], env, "delta_o") if own_output else None
        if own_output:
            self.o_weight = None

    @staticmethod
    def tensor_needs(spec: GatedDeltaSpec) -> List[TensorNeed]:
        s = spec
        kd, vd, hd = s.n_kv_heads * s.head_dim, s.n_heads * s.v_head_dim, s.n_heads * s.head_dim
        return [TensorNeed(s.q_proj, (kd, s.hidden)), TensorNeed(s.k_proj, (kd, s.hidden)), TensorNeed(s.v_proj, (vd, s.hidden)),
                TensorNeed(s.q_conv, (kd, s.conv_taps)), TensorNeed(s.k_conv, (kd, s.conv_taps)),
                TensorNeed(s.v_conv, (vd, s.conv_taps)), TensorNeed(s.beta_proj, (s.n_heads, s.hidden)),
                TensorNeed(s.decay_in, (s.decay_rank, s.hidden)), TensorNeed(s.decay_out, (hd, s.decay_rank)),
                TensorNeed(s.decay_bias, (hd,)), TensorNeed(s.decay_log, (s.n_heads,)),
                TensorNeed(s.gate_in, (s.gate_rank, s.hidden)), TensorNeed(s.gate_out, (vd, s.gate_rank)),
                TensorNeed(s.out_norm, (s.v_head_dim,)), TensorNeed(s.o_proj, (s.hidden, vd))]

    def kv_need(self) -> Optional[GroupKey]:
        return None

    def state_need(self) -> Dict[str, StateNeed]:
        s, pre = self.spec, self.state_prefix
        return {pre + "S": StateNeed((s.n_heads, s.v_head_dim, s.head_dim), torch.float32),
                pre + "conv": self.conv.state_need()}

    def context_into(self, x: torch.Tensor, step, memory: int, writes: bool, out: torch.Tensor, scale: float = 1.0,
                     proj: Optional[torch.Tensor] = None) -> None:
        s, ws, pre = self.spec, self.env.workspace, self.state_prefix
        n = x.shape[0]
        if not writes:
            raise ValueError("a recurrent mixer advances its own state; it cannot read another run's")
        if proj is None:
            proj = self.proj.forward(x, out_dtype=torch.float32, tag=pre + "delta_in")
        c_qkv = 2 * self.kd + self.vd
        bounds = (0, c_qkv, c_qkv + s.n_heads, c_qkv + s.n_heads + self.ra, c_qkv + s.n_heads + self.ra + self.rg)
        qkv, beta, a_in, g_in = ws.columns(proj, bounds)
        dt = self.decay_out.forward(a_in, tag=pre + "delta_dt")
        gate = self.gate_out.forward(g_in, tag=pre + "delta_gate")
        conved = ws.get(pre + "delta_conved", n, c_qkv, torch.float32)
        self.conv.forward(qkv, conved, state_tensor(step, memory, pre + "conv"), step)
        q, k, v = ws.columns(conved, (0, self.kd, 2 * self.kd, c_qkv))
        o = ws.get(pre + "delta_readout", n, self.vd, torch.float32)
        seq_ops.gated_recurrence(seq_ops.DELTA, q, k, v, o, state_tensor(step, memory, pre + "S"), step, s.n_heads,
                                 s.n_kv_heads, s.head_dim, s.v_head_dim, dt_in=dt, beta=beta, a_log=self.a_log,
                                 dt_bias=self.dt_bias, unit_eps=s.unit_eps)
        seq_ops.head_norm_gate(o, self.norm_gain, gate, out, s.n_heads, s.v_head_dim, s.norm_eps, scale)

    def forward(self, x: torch.Tensor, step, memory: int, writes: bool = True) -> torch.Tensor:
        ctx = self.env.workspace.get(self.state_prefix + "delta_ctx", x.shape[0], self.context_width, self.env.dtype)
        self.context_into(x, step, memory, writes, ctx)
        return self.o.forward(ctx, tag="delta_o", slices_ok=True)


class Hgrn2:
    @staticmethod
    def kernel_libraries(spec, dtype):
        return ("sequence",)

    def __init__(self, spec: Hgrn2Spec, weights, env: BuildEnv, own_output: bool = True, own_input: bool = True):
        s = spec
        self.spec, self.env = spec, env
        self.state_prefix = ""
        self.hd, self.vd = s.n_heads * s.head_dim, s.n_heads * s.v_head_dim
        self.context_width = self.vd
        mats = [weights.get(s.q_proj), weights.get(s.f_proj), weights.get(s.v_proj)]
        self.input_matrices = None if own_input else mats
        self.input_width = sum(int(m.shape[0]) for m in mats)
        self.proj = Linear(mats, env, "hgrn2_in") if own_input else None
        self.f_bias = _vec(weights, s.f_bias, env) if s.f_bias else None      # added inside the recurrence's kernel
        self.lower = _vec(weights, s.lower, env)
        self.norm_gain = _vec(weights, s.out_norm, env)
        self.o_weight = weights.get(s.o_proj)
        self.o = Linear([self.o_weight], env, "hgrn2_o") if own_output else None
        if own_output:
            self.o_weight = None

    @staticmethod
    def tensor_needs(spec: Hgrn2Spec) -> List[TensorNeed]:
        s = spec
        hd, vd = s.n_heads * s.head_dim, s.n_heads * s.v_head_dim
        needs = [TensorNeed(s.q_proj, (hd, s.hidden)), TensorNeed(s.f_proj, (hd, s.hidden)), TensorNeed(s.lower, (hd,)),
                 TensorNeed(s.v_proj, (vd, s.hidden)), TensorNeed(s.out_norm, (s.v_head_dim,)), TensorNeed(s.o_proj, (s.hidden, vd))]
        if s.f_bias:
            needs.append(TensorNeed(s.f_bias, (hd,)))
        return needs

    def kv_need(self) -> Optional[GroupKey]:
        return None

    def state_need(self) -> Dict[str, StateNeed]:
        s = self.spec
        return {self.state_prefix + "S": StateNeed((s.n_heads, s.v_head_dim, s.head_dim), torch.float32)}

    def context_into(self, x: torch.Tensor, step, memory: int, writes: bool, out: torch.Tensor, scale: float = 1.0,
                     proj: Optional[torch.Tensor] = None) -> None:
        s, ws, pre = self.spec, self.env.workspace, self.state_prefix
        n = x.shape[0]
        if not writes:
            raise ValueError("a recurrent mixer advances its own state; it cannot read another run's")
        if proj is None:
            proj = self.proj.forward(x, out_dtype=torch.float32, tag=pre + "hgrn2_in")
        q, f, v = ws.columns(proj, (0, self.hd, 2 * self.hd, 2 * self.hd + self.vd))
        o = ws.get(pre + "hgrn2_readout", n, self.vd, torch.float32)
        seq_ops.gated_recurrence(seq_ops.FORGET, q, f, v, o, state_tensor(step, memory, pre + "S"), step, s.n_heads,
                                 s.n_heads, s.head_dim, s.v_head_dim, lower=self.lower, f_bias=self.f_bias)
        seq_ops.head_norm_gate(o, self.norm_gain, None, out, s.n_heads, s.v_head_dim, s.norm_eps, scale)

    def forward(self, x: torch.Tensor, step, memory: int, writes: bool = True) -> torch.Tensor:
        ctx = self.env.workspace.get(self.state_prefix + "hgrn2_ctx", x.shape[0], self.context_width, self.env.dtype)
        self.context_into(x, step, memory, writes, ctx)
        return self.o.forward(ctx, tag="hgrn2_o", slices_ok=True)


class Mamba2:
    @staticmethod
    def kernel_libraries(spec, dtype):
        return ("sequence",)

    def __init__(self, spec: Mamba2Spec, weights, env: BuildEnv):
        s = spec
        if s.n_heads % s.groups:
            raise ValueError("mamba2: heads must be a multiple of the groups of B and C")
        self.inner, self.gn = s.n_heads * s.v_head_dim, s.groups * s.state
        if self.inner % s.norm_groups:
            raise ValueError(f"mamba2: rows of {self.inner} do not split into {s.norm_groups} equal parts for the norm")
        self.spec, self.env = spec, env
        self.channels = self.inner + 2 * self.gn
        self.proj = Linear([weights.get(s.in_proj)], env, "mamba_in")
        self.conv = ShortConv([weights.get(s.conv)], env, silu=True, name="mamba_conv",
                              bias=weights.get(s.conv_bias) if s.conv_bias else None)
        if self.conv.channels != self.channels:
            raise ValueError(f"mamba2: the convolution has {self.conv.channels} channels, xs, B and C have {self.channels}")
        self.a_log, self.dt_bias, self.skip = (_vec(weights, n, env) for n in (s.a_log, s.dt_bias, s.d_skip))
        self.norm_weight = _vec(weights, s.out_norm, env)
        self.o = Linear([weights.get(s.o_proj)], env, "mamba_o")

    @staticmethod
    def tensor_needs(spec: Mamba2Spec) -> List[TensorNeed]:
        s = spec
        inner, gn = s.n_heads * s.v_head_dim, s.groups * s.state
        needs = [TensorNeed(s.in_proj, (2 * inner + 2 * gn + s.n_heads, s.hidden)),
                 TensorNeed(s.conv, (inner + 2 * gn, s.conv_taps))]
        if s.conv_bias:
            needs.append(TensorNeed(s.conv_bias, (inner + 2 * gn,)))
        needs += [TensorNeed(s.dt_bias, (s.n_heads,)), TensorNeed(s.a_log, (s.n_heads,)), TensorNeed(s.d_skip, (s.n_heads,)),
                  TensorNeed(s.out_norm, (inner,)), TensorNeed(s.o_proj, (s.hidden, inner))]
        return needs

    def kv_need(self) -> Optional[GroupKey]:
        return None

    def state_need(self) -> Dict[str, StateNeed]:
        s = self.spec
        return {"S": StateNeed((s.n_heads, s.v_head_dim, s.state), torch.float32), "conv": self.conv.state_need()}

    def forward(self, x: torch.Tensor, step, memory: int, writes: bool = True) -> torch.Tensor:
        s, ws = self.spec, self.env.workspace
        n = x.shape[0]
        if not writes:
            raise ValueError("a recurrent mixer advances its own state; it cannot read another run's")
        proj = self.proj.forward(x, out_dtype=torch.float32, tag="mamba_in")
        z, xbc, dt = ws.columns(proj, (0, self.inner, self.inner + self.channels, self.inner + self.channels + s.n_heads))
        conved = ws.get("mamba_conved", n, self.channels, torch.float32)
        self.conv.forward(xbc, conved, state_tensor(step, memory, "conv"), step)
        xs, b, c = ws.columns(conved, (0, self.inner, self.inner + self.gn, self.channels))
        y = ws.get("mamba_readout", n, self.inner, torch.float32)
        seq_ops.gated_recurrence(seq_ops.SSD, c, b, xs, y, state_tensor(step, memory, "S"), step, s.n_heads, s.groups,
                                 s.state, s.v_head_dim, dt_in=dt, a_log=self.a_log, dt_bias=self.dt_bias, skip=self.skip)
        ctx = ws.get("mamba_ctx", n, self.inner, self.env.dtype)
        seq_ops.gated_group_norm(y, z, self.norm_weight, ctx, s.norm_groups, s.norm_eps)
        return self.o.forward(ctx, tag="mamba_o", slices_ok=True)


register("mixer", "gated_delta", GatedDelta)
register("mixer", "mamba2", Mamba2)
register("mixer", "hgrn2", Hgrn2)
