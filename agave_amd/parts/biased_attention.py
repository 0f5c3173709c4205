"""Softmax attention with a bias on the scores by distance, as a mixer.

In the order of its steps: q, k, v (and the gate's logits) in one product; k and v rows appended to
the cache as they are (there is no rotation and no norm: positions enter through the bias and the
mask alone); scores ``scale * q.k`` plus the bias of the distance ``i - j``; the keys ``j <= i`` with
``i - j < window`` or ``j < keep_first``; softmax, with ``exp(sink_h)`` added to the denominator where the
mixer has sinks; the heads' outputs times ``sigmoid(gate)`` element by element where it has a gate; the
output product.

The bias is either a slope per head (``-slope_h (i - j)``) or a learned table over buckets of distances;
the buckets are folded into a table over distances once at load (one column per distance up to the one
from which the last bucket holds), so the kernels know a slope or a table and nothing of buckets.

A mixer without key and value projections appends nothing and reads the memory that its run-order
entry names (another layer's keys and values as the cache holds them), through its own mask.

A mixer may besides have biases on its q, k and v products, an RMS norm over the whole row of q and of k (all heads
side by side) followed by a rotation of each head's first elements, a cap on the scaled scores, and chunks of
positions instead of (or besides) a window.  With a norm or a rotation the first product leaves 32-bit rows, and one
kernel norms, rotates and rounds them to the engine's element type once.

Scores, bias, softmax and the sums over the values are 32-bit in both engines.
"""
from __future__ import annotations

import math
from typing import List, Optional

import torch

from ..cache import GroupKey, StateNeed
from ..config.spec import BiasedAttentionSpec, ScoreBiasSpec
from ..ops import attention_biased as ops
from ..ops import kernels
from ..weights.loader import TensorNeed
from .base import BuildEnv, lookup, register
from .linear import Linear


def bucket_of_distance(n: int, buckets: int, max_distance: int) -> int:
    """Distances below half the buckets have a bucket each; beyond, buckets grow evenly in the logarithm of
    the distance up to ``max_distance``, and the last bucket takes everything farther.  The logarithms are
    taken in double precision; a quotient within 1e-9 of a whole number counts as that number."""
    half = buckets // 2
    if n < half:
        return n
    x = math.log(n / half) / math.log(max_distance / half) * (buckets - half)
    near = round(x)
    steps = near if abs(x - near) < 1e-9 else math.floor(x)
    return min(buckets - 1, half + int(steps))


def distance_table(table: torch.Tensor, buckets: int, max_distance: int) -> torch.Tensor:
    """[heads, distances] float32 from a learned [buckets, heads]: column n holds the bias of distance n, the
    last column that of every distance from there on."""
    half = buckets // 2
    if half < 1 or max_distance <= half:
        raise ValueError(f"a bias over {buckets} buckets needs a largest distance above {half}, got {max_distance}")
    last = 0
    while bucket_of_distance(last, buckets, max_distance) < buckets - 1:
        last += 1
        if last > max(max_distance, buckets) + 1:
            raise ValueError("the buckets of distances never reach the last one")
    idx = torch.tensor([bucket_of_distance(n, buckets, max_distance) for n in range(last + 1)], dtype=torch.long)
    return table.to(torch.float32)[idx].t().contiguous()


class BiasedAttention:
    @staticmethod
    def kernel_libraries(spec, dtype):
        return ("attention_biased",)

    def __init__(self, spec: BiasedAttentionSpec, weights, env: BuildEnv):
        s = spec
        if s.n_heads % s.n_kv_heads:
            raise ValueError("query heads must be a multiple of kv heads")
        if bool(s.k_proj) != bool(s.v_proj):
            raise ValueError("biased attention: key and value projections come together or not at all")
        self.spec, self.env = spec, env
        self.qd, self.kd, self.vd = s.n_heads * s.head_dim, s.n_kv_heads * s.head_dim, s.n_kv_heads * s.v_head_dim
        self.ctx = s.n_heads * s.v_head_dim
        self.own_kv = bool(s.k_proj)
        def bias(name):
            return weights.get(name) if name else None
        mats, biases = [weights.get(s.q_proj)], [bias(s.q_bias)]
        bounds = [0, self.qd]
        if self.own_kv:
            mats += [weights.get(s.k_proj), weights.get(s.v_proj)]
            biases += [bias(s.k_bias), bias(s.v_bias)]
            bounds += [bounds[-1] + self.kd, bounds[-1] + self.kd + self.vd]
        elif s.k_bias or s.v_bias or s.k_row_norm is not None:
            raise ValueError("biased attention: a mixer without key and value projections has no biases or norm for them")
        if s.gate_proj:
            mats.append(weights.get(s.gate_proj))
            biases.append(None)
            bounds.append(bounds[-1] + self.ctx)
        self._bounds = tuple(bounds)
        # the norm over whole rows and the rotation: q and k pass a kernel of their own on their way
        self.q_weight = self.k_weight = None
        self.q_eps = self.k_eps = 0.0
        for which, ns, size in (("q", s.q_row_norm, self.qd), ("k", s.k_row_norm, self.kd)):
            if ns is None:
                continue
            if ns.kind != "rmsnorm" or ns.size != size or ns.bias:
                raise ValueError(f"biased attention: the norm over the {which} rows must be an RMS norm of {size} elements")
            w = weights.get(ns.weight).to(torch.float32)
            w = (w + 1.0 if ns.add_one else w).contiguous().to(env.device)
            if which == "q":
                self.q_weight, self.q_eps = w, float(ns.eps)
            else:
                self.k_weight, self.k_eps = w, float(ns.eps)
        self.position = lookup("position", s.position.kind)(s.position, env)
        table = getattr(self.position, "rotation_table", None)
        if table is None:
            raise ValueError(f"biased attention: the position encoding {s.position.kind!r} is no rotation of pairs")
        self.freq, interleaved = table()
        if interleaved:
            raise ValueError("biased attention: rotated pairs are (e, e + rotary_dim / 2)")
        self.magnitude = float(getattr(self.position, "magnitude", 1.0))
        self.prepares_rows = self.q_weight is not None or self.k_weight is not None or self.freq is not None
        # one product for everything that reads the mixer's input; its biases are added by the kernel that prepares the
        # rows where there is one, else by the product
        self.row_biases = (None, None, None)
        if self.prepares_rows:
            def vec(b):
                return b.to(torch.float32).contiguous().to(env.device) if b is not None else None
            self.row_biases = (vec(biases[0]), vec(biases[1]) if self.own_kv else None, vec(biases[2]) if self.own_kv else None)
            biases = None
        self.proj = Linear(mats, env, "qkvg", biases=biases)
        if s.chunk is not None and s.keep_first:
            raise ValueError("biased attention: chunks go without kept first positions")
        self.o = Linear([weights.get(s.o_proj)], env, "attn_o")
        self.sink = weights.get(s.sink).to(torch.float32).contiguous().to(env.device) if s.sink else None
        b = s.bias
        if b.kind == "none":
            self.bias_mode, self.bias = ops.BIAS_NONE, None
        elif b.kind == "slopes":
            slopes = [2.0 ** (-b.slope_log2 * (h + 1) / s.n_heads) for h in range(s.n_heads)]
            self.bias_mode, self.bias = ops.BIAS_SLOPES, torch.tensor(slopes, dtype=torch.float32, device=env.device)
        elif b.kind == "buckets":
            self.bias_mode = ops.BIAS_TABLE
            self.bias = distance_table(weights.get(b.table), b.buckets, b.max_distance).to(env.device)
        else:
            raise ValueError(f"biased attention: unknown kind of bias {b.kind!r} (none, slopes, buckets)")

    @staticmethod
    def tensor_needs(spec: BiasedAttentionSpec) -> List[TensorNeed]:
        s = spec
        qd, kd, vd, ctx = s.n_heads * s.head_dim, s.n_kv_heads * s.head_dim, s.n_kv_heads * s.v_head_dim, s.n_heads * s.v_head_dim
        needs = [TensorNeed(s.q_proj, (qd, s.hidden))]
        if s.k_proj:
            needs += [TensorNeed(s.k_proj, (kd, s.hidden)), TensorNeed(s.v_proj, (vd, s.hidden))]
        if s.bias.kind == "buckets":
            needs.append(TensorNeed(s.bias.table, (s.bias.buckets, s.n_heads)))
        if s.sink:
            needs.append(TensorNeed(s.sink, (s.n_heads,)))
        if s.gate_proj:
            needs.append(TensorNeed(s.gate_proj, (ctx, s.hidden)))
        needs.append(TensorNeed(s.o_proj, (s.hidden, ctx)))
        for name, size in ((s.q_bias, qd), (s.k_bias, kd), (s.v_bias, vd)):
            if name:
                needs.append(TensorNeed(name, (size,)))
        for ns in (s.q_row_norm, s.k_row_norm):
            if ns is not None:
                needs.append(TensorNeed(ns.weight, (ns.size,)))
        return needs

    def kv_need(self) -> Optional[GroupKey]:
        s = self.spec
        return GroupKey(s.window, s.n_kv_heads, s.head_dim, chunk=s.chunk, v_head_dim=s.v_head_dim, layout="rows_vt",
                        keep_first=s.keep_first if s.window is not None else 0)

    def state_need(self) -> Optional[StateNeed]:
        return None

    def forward(self, x: torch.Tensor, step, memory: int, writes: bool = True) -> torch.Tensor:
        s, ws = self.spec, self.env.workspace
        n = x.shape[0]
        if writes != self.own_kv:
            raise ValueError("biased attention: a mixer with key and value projections appends to its memory, one "
                             "without reads another's; the run order says otherwise")
        group = step.cache.group_of_memory[memory]
        k_pages, v_pages, packed = step.cache.pages_of(memory)
        table, base = step.tables[group]
        head = step.cache.group_keys[group].kept_pages
        if self.prepares_rows:
            # 32-bit rows from the product; norm, rotation and the one rounding to the engine's type in one kernel
            proj = self.proj.forward(x, out_dtype=torch.float32, tag="qkvg32")
            cols = ws.columns(proj, self._bounds)
            q = ws.get("attn_q_rows", n, self.qd, x.dtype)
            k = v = None                                        # (k and v go straight into the cache pages)
            ops.row_norm_rope(cols[0], cols[1] if self.own_kv else None, cols[2] if self.own_kv else None, q, None, None,
                              self.q_weight, self.k_weight, self.q_eps, self.k_eps, self.freq, self.magnitude, step,
                              s.n_heads, s.n_kv_heads, s.head_dim, s.v_head_dim, biases=self.row_biases,
                              pages=(k_pages, v_pages, table, base, head, packed) if self.own_kv else None)
            gate = None
            if s.gate_proj:
                g32 = cols[3 if self.own_kv else 1]
                gate = ws.get("attn_gate_rows", n, self.ctx, x.dtype)
                kernels.cast(g32, gate)
        else:
            proj = self.proj.forward(x, tag="qkvg")
            cols = ws.columns(proj, self._bounds)
            q = cols[0]
            k, v = (cols[1], cols[2]) if self.own_kv else (None, None)
            gate = cols[3 if self.own_kv else 1] if s.gate_proj else None
        if self.own_kv and k is not None:
            ops.kv_append_rows(k, v, k_pages, v_pages, table, base, head, step, s.n_kv_heads, s.head_dim,
                               s.v_head_dim, packed)
        ctx = ws.get("attn_ctx", n, self.ctx, x.dtype)
        ops.attention(q, ctx, gate, k_pages, v_pages, table, base, head, step, s.n_heads, s.n_kv_heads, s.head_dim,
                      s.v_head_dim, s.scale, s.window, s.keep_first, self.bias_mode, self.bias, self.sink, packed,
                      workspace=ws, chunk=s.chunk, softcap=s.softcap)
        return self.o.forward(ctx, tag="attn_o", slices_ok=True)       # the block adds it to the residual stream


register("mixer", "biased_attention", BiasedAttention)
