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

A step of many rows in which every sequence starts at its first position (a prompt that comes whole, or its first
piece) needs nothing of the cache, and there the folded form would multiply every score over ``kv_rank + rot_dim``
elements and every sum over ``kv_rank``, several times what the heads' own sizes ask for.  Such a step makes every
head's keys ``[W_uk,h c | r]`` and values ``W_uv,h c`` of its own tokens with two products, writes them into pages of
its own that live as long as the step, and runs the attention with a key head per query head (``fresh_prompt``; in
bfloat16, where the heads' sizes are ones the matrix cores take).  The cache is written as always, so whatever comes
after the step reads the latent rows.  Both forms compute the same sums in another order.

A mixer without a latent projection of its own appends nothing and reads the rows of the memory that its run-order
entry names, with its own ``W_uk``, ``W_uv`` and queries.

Norm sums, angles, scores, softmax and the sums over the cached rows are 32-bit in both engines.
"""
from __future__ import annotations

from typing import List, Optional

import numpy as np
import torch

from ..cache import PAGE, GroupKey, StateNeed
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
        # the products of the form that makes every head's keys and values (prompts from their first position on)
        self.fresh_min_rows = 64
        self.fresh_ok = (env.dtype == torch.bfloat16 and self.qd % 8 == 0 and self.qd <= 256 and s.v_head_dim % 16 == 0
                         and s.v_head_dim <= 256 and s.kv_rank % 8 == 0)
        if self.fresh_ok:
            self.k_up = Linear([weights.get(s.k_up)], env, "latent_k_up")
            self.v_up_all = Linear([weights.get(s.v_up)], env, "latent_v_up")
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
            k_row = ws.get(f"latent_row_{memory}", n, self.kd, x.dtype)    # (of its own: later layers of this step may read it)
            ops.latent_prepare(cols[0], self.q_weight, cq, cols[1], self.kv_weight, k_row, s.kv_rank, s.rot_dim, self.freq,
                               step, s.norm_eps)
            c_cols = ws.columns(k_row, (0, s.kv_rank))[0]
            attn_ops.kv_append_rows(k_row, c_cols, k_pages, v_pages, table, base, 0, step, 1, self.kd, s.kv_rank, packed)
            at = 2
        else:
            ops.latent_prepare(cols[0], self.q_weight, cq, None, None, None, s.kv_rank, s.rot_dim, None, step, s.norm_eps)
        gate = cols[at] if s.gate_proj else None
        q = self.q_up.forward(cq, tag="latent_q")
        notes = step.__dict__.setdefault("latent_rows", {})          # this step's latent rows, by memory
        if self.own_kv:
            notes[memory] = k_row
        ctx = ws.get("attn_ctx", n, self.ctx, x.dtype)
        if self.fresh_ok and not step.is_decode and n >= self.fresh_min_rows and not any(step.pos0) and memory in notes:
            self.fresh_prompt(q, notes[memory], gate, ctx, step)
            return self.o.forward(ctx, tag="attn_o", slices_ok=True)
        folded = ws.get("latent_folded", n, s.n_heads * self.kd, x.dtype)
        ops.heads_product(q, self.fold, folded, s.n_heads, self.qd, self.kd, tail=s.rot_dim, freq=self.freq,
                          tok_pos=step.tok_pos)
        mixed = ws.get("latent_mixed", n, s.n_heads * s.kv_rank, x.dtype)
        attn_ops.attention(folded, mixed, None, k_pages, v_pages, table, base, 0, step, s.n_heads, 1, self.kd, s.kv_rank,
                           s.scale, None, 0, attn_ops.BIAS_NONE, None, None, packed, workspace=ws)
        ops.heads_product(mixed, self.v_up, ctx, s.n_heads, s.kv_rank, s.v_head_dim, gate=gate)
        return self.o.forward(ctx, tag="attn_o", slices_ok=True)       # the block adds it to the residual stream

    def fresh_prompt(self, q: torch.Tensor, k_row: torch.Tensor, gate: Optional[torch.Tensor], ctx: torch.Tensor, step) -> None:
        """Every sequence of the step starts at position 0: the heads' own keys and values of the step's tokens, in
        pages that belong to the step (sequence b holds ``ceil(n_b / 64)`` of them, one after another), and the
        attention over those."""
        s, ws = self.spec, self.env.workspace
        n, heads = q.shape[0], s.n_heads
        plan = step.__dict__.get("fresh_pages")
        if plan is None:
            counts = [-(-c // PAGE) for c in (b - a for a, b in zip(step.cu[:-1], step.cu[1:]))]
            width = max(counts)
            rows = np.zeros((step.n_seqs, width), dtype=np.int32)
            at = 0
            for b, c in enumerate(counts):
                rows[b, :c] = np.arange(at, at + c, dtype=np.int32)
                at += c
            table = torch.from_numpy(rows).to(self.env.device)
            plan = step.__dict__["fresh_pages"] = (table, torch.zeros(step.n_seqs, dtype=torch.int32, device=self.env.device), at)
        table, base, n_pages = plan
        c_rows = ws.columns(k_row, (0, s.kv_rank))[0]
        k_plain = self.k_up.forward(c_rows, tag="latent_k_plain")
        values = self.v_up_all.forward(c_rows, tag="latent_values")
        k_full = ws.get("latent_k_full", n, heads * self.qd, q.dtype)
        ops.latent_expand(q, k_plain, k_row, s.kv_rank, k_full, heads, s.head_dim, s.rot_dim, self.freq, step.tok_pos)
        hd_k = (self.qd + 31) // 32 * 32
        before = ws.allocations
        k_pages = ws.get("latent_fresh_k", n_pages, heads * PAGE * hd_k, q.dtype)
        v_pages = ws.get("latent_fresh_v", n_pages, heads * s.v_head_dim * PAGE, q.dtype)
        if ws.allocations != before or hd_k != self.qd:
            # (new memory may hold anything, and a place that no token writes must not hold what is no number; the
            # lanes of a key step past the head's end must hold zeros)
            k_pages.zero_()
            v_pages.zero_()
        k_pages = k_pages.view(n_pages, heads, PAGE, hd_k)
        v_pages = v_pages.view(n_pages, heads, s.v_head_dim, PAGE)
        attn_ops.kv_append_rows(k_full, values, k_pages, v_pages, table, base, 0, step, heads, self.qd, s.v_head_dim, True)
        attn_ops.attention(q, ctx, None, k_pages, v_pages, table, base, 0, step, heads, heads, self.qd, s.v_head_dim,
                           s.scale, None, 0, attn_ops.BIAS_NONE, None, None, True)
        if gate is not None:
            ops.gate_rows(ctx, gate)


register("mixer", "latent_attention", LatentAttention)
