"""Attention whose keys and values are made from one small latent row per position, as a mixer.

The cache holds, per position, the row ``[c | r]``: the normed latent ``c`` (``kv_rank`` elements) and the rotated
key part ``r`` (``rot_dim`` elements) that all heads share; nothing per head.  Head h's key would be
``[W_uk,h c | r]`` and its value ``W_uv,h c``.  Neither is ever made.  Since ``q . (W_uk,h c) = (W_uk,h^T q) . c``, each
head's plain query part is folded through its key matrix once per token, and the attention then runs with one key
head for all query heads, directly on the cached rows: keys ``[c | r]``, values ``c``; head h's sum over latent rows
is turned into its values by ``W_uv,h`` afterwards (the softmax weights add up to one, so the sum commutes with the
matrix).  The cache is read once for all heads and holds ``kv_rank + rot_dim`` numbers a position.

In the order of its steps: one product for the query latent, the key/value latent and the gate's logits (32-bit
rows out); the latents' norms and the rotation of ``r`` (``latent_prepare``), the row appended to the cache; the query
product; per head the fold through ``W_uk`` and the rotation of the query's last ``rot_dim`` elements
(``heads_product``); the attention; per head ``W_uv`` and the gate (``heads_product``); the output product.

A mixer without a latent projection of its own appends nothing and reads the rows of the memory that its run-order
entry names, with its own ``W_uk``, ``W_uv`` and queries.

Norm sums, angles, scores, softmax and the sums over the cached rows are 32-bit in both engines.
"""
from __future__ import annotations

from typing import List, Optional

import torch

from ..cache import GroupKey, StateNeed
from ..config.spec import LatentAttentionSpec
from ..ops import attention_biased as attn_ops
from ..ops import latent as ops
from ..weights.loader import TensorNeed
from .base import BuildEnv, lookup, register
from .linear import Linear


class LatentAttention:
    @staticmethod
    def kernel_libraries(spec, dtype):
        return ("latent", "attention_biased")

    def __init__(self, spec: LatentAttentionSpec, weights, env: BuildEnv):
        s = spec
        if bool(s.kv_down) != bool(s.kv_norm):
            raise ValueError("latent attention: the key/value latent's projection and norm come together or not at all")
        if min(s.n_heads, s.head_dim, s.v_head_dim, s.q_rank, s.kv_rank) < 1 or s.rot_dim < 0:
            raise ValueError("latent attention: sizes must be positive")
        self.spec, self.env = spec, env
        self.own_kv = bool(s.kv_down)
        self.qd = s.head_dim + s.rot_dim                # a head of the query product
        self.kd = s.kv_rank + s.rot_dim                 # a cached row, and a head of the folded query
        self.ctx = s.n_heads * s.v_head_dim
        mats = [weights.get(s.q_down)]
        bounds = [0, s.q_rank]
        if self.own_kv:
            mats.append(weights.get(s.kv_down))
            bounds.append(bounds[-1] + self.kd)
        if s.gate_proj:
            mats.append(weights.get(s.gate_proj))
            bounds.append(bounds[-1] + self.ctx)
        self._bounds = tuple(bounds)
        self.proj = Linear(mats, env, "latent_in")      # everything that reads the mixer's input, one product
        self.q_up = Linear([weights.get(s.q_up)], env, "latent_q")
        self.o = Linear([weights.get(s.o_proj)], env, "attn_o")
        dev = env.device
        self.q_weight = weights.get(s.q_norm).to(torch.float32).contiguous().to(dev)
        self.kv_weight = weights.get(s.kv_norm).to(torch.float32).contiguous().to(dev) if self.own_kv else None
        # per head: W_uk,h^T [kv_rank, head_dim] (the fold of the query) and W_uv,h [v_head_dim, kv_rank]
        uk = weights.get(s.k_up).to(env.dtype).view(s.n_heads, s.head_dim, s.kv_rank)
        self.fold = uk.transpose(1, 2).contiguous().to(dev)
        self.v_up = weights.get(s.v_up).to(env.dtype).view(s.n_heads, s.v_head_dim, s.kv_rank).contiguous().to(dev)
        self.freq = None
        if s.rot_dim and s.position.kind != "none":
            if s.position.interleaved:
                raise ValueError("latent attention: the rotation pairs element i with i + rotary_dim / 2")
            if s.position.rotary_dim > s.rot_dim:
                raise ValueError(f"latent attention: {s.position.rotary_dim} rotated elements exceed rot_dim ({s.rot_dim})")
            freq, _ = lookup("position", s.position.kind)(s.position, env).fused_rotation()
            self.freq = freq.contiguous() if freq is not None else None

    @staticmethod
    def tensor_needs(spec: LatentAttentionSpec) -> List[TensorNeed]:
        s = spec
        qd, ctx = s.head_dim + s.rot_dim, s.n_heads * s.v_head_dim
        needs = [TensorNeed(s.q_down, (s.q_rank, s.hidden)), TensorNeed(s.q_norm, (s.q_rank,)),
                 TensorNeed(s.q_up, (s.n_heads * qd, s.q_rank))]
        if s.kv_down:
            needs += [TensorNeed(s.kv_down, (s.kv_rank + s.rot_dim, s.hidden)), TensorNeed(s.kv_norm, (s.kv_rank,))]
        needs += [TensorNeed(s.k_up, (s.n_heads * s.head_dim, s.kv_rank)), TensorNeed(s.v_up, (ctx, s.kv_rank))]
        if s.gate_proj:
            needs.append(TensorNeed(s.gate_proj, (ctx, s.hidden)))
        needs.append(TensorNeed(s.o_proj, (s.hidden, ctx)))
        return needs

    def kv_need(self) -> Optional[GroupKey]:
        s = self.spec
        # one key head: rows [c | r]; the values are the rows' first kv_rank elements, kept transposed inside a page
        # as the attention kernel reads them
        return GroupKey(None, 1, self.kd, v_head_dim=s.kv_rank, layout="rows_vt")

    def state_need(self) -> Optional[StateNeed]:
        return None

    def forward(self, x: torch.Tensor, step, memory: int, writes: bool = True) -> torch.Tensor:
        s, ws = self.spec, self.env.workspace
        n = x.shape[0]
        if writes != self.own_kv:
            raise ValueError("latent attention: a mixer with a key/value latent of its own appends to its memory, one "
                             "without reads another's; the run order says otherwise")
        group = step.cache.group_of_memory[memory]
        k_pages, v_pages, packed = step.cache.pages_of(memory)
        table, base = step.tables[group]
        proj = self.proj.forward(x, out_dtype=torch.float32, tag="latent_in")
        cols = ws.columns(proj, self._bounds)
        at = 1
        cq = ws.get("latent_cq", n, s.q_rank, x.dtype)
        if self.own_kv:
            k_row = ws.get("latent_row", n, self.kd, x.dtype)
            ops.latent_prepare(cols[0], self.q_weight, cq, cols[1], self.kv_weight, k_row, s.kv_rank, s.rot_dim, self.freq,
                               step, s.norm_eps)
            c_cols = ws.columns(k_row, (0, s.kv_rank))[0]
            attn_ops.kv_append_rows(k_row, c_cols, k_pages, v_pages, table, base, 0, step, 1, self.kd, s.kv_rank, packed)
            at = 2
        else:
            ops.latent_prepare(cols[0], self.q_weight, cq, None, None, None, s.kv_rank, s.rot_dim, None, step, s.norm_eps)
        gate = cols[at] if s.gate_proj else None
        q = self.q_up.forward(cq, tag="latent_q")
        folded = ws.get("latent_folded", n, s.n_heads * self.kd, x.dtype)
        ops.heads_product(q, self.fold, folded, s.n_heads, self.qd, self.kd, tail=s.rot_dim, freq=self.freq,
                          tok_pos=step.tok_pos)
        mixed = ws.get("latent_mixed", n, s.n_heads * s.kv_rank, x.dtype)
        attn_ops.attention(folded, mixed, None, k_pages, v_pages, table, base, 0, step, s.n_heads, 1, self.kd, s.kv_rank,
                           s.scale, None, 0, attn_ops.BIAS_NONE, None, None, packed, workspace=ws)
        ctx = ws.get("attn_ctx", n, self.ctx, x.dtype)
        ops.heads_product(mixed, self.v_up, ctx, s.n_heads, s.kv_rank, s.v_head_dim, gate=gate)
        return self.o.forward(ctx, tag="attn_o", slices_ok=True)       # the block adds it to the residual stream


register("mixer", "latent_attention", LatentAttention)
