"""Python faces of ``csrc/sequence.hip``: the short convolution, the head norm with rotation and
cache rows, the attention with talking heads, the gated linear recurrence and the read-out norm.

Every function checks on the host what its kernel and grid assume and launches on the current
stream.  Rows between a mixer's first product and its output product are float32 here; the cache
pages and the rows handed to the output product have the engine's element type.
"""
from __future__ import annotations

import ctypes
from typing import Optional

import torch

from . import kernels, library
from .kernels import _P, _I, _L, _F, _dev, _f32vec, _i32, dt, ptr, stream

LIBRARY = "sequence"

kernels.register_signatures(LIBRARY, {
    "agave_short_conv": [_P, _L, _P, _P, _P, _L, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P, _P],
    "agave_head_norm_rope_rows": [_I, _P, _L, _P, _L, _P, _L, _P, _L, _P, _P, _F, _F, _I, _I, _P, _I, _I, _P, _P,
                                  _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _I, _P],
    "agave_talk_attention": [_I, _P, _L, _P, _L, _P, _L, _P, _P, _P, _I, _P, _I, _P, _P, _P, _I, _I, _I, _I, _I,
                             _F, _I, _F, _P, _I, _P],
    "agave_gated_recurrence": [_I, _P, _L, _P, _L, _P, _L, _P, _L, _P, _L, _P, _P, _P, _P, _P, _P, _L, _P, _P, _P,
                               _I, _I, _I, _I, _I, _F, _I, _P],
    "agave_gated_group_norm": [_I, _P, _L, _P, _L, _P, _P, _L, _I, _I, _I, _F, _P],
    "agave_head_norm_gate": [_I, _P, _L, _P, _P, _L, _P, _L, _I, _I, _I, _F, _F, _P],
    "agave_scaled_sum": [_I, _P, _L, _F, _P, _L, _F, _P, _L, _I, _I, _P],
})

MAX_TAPS = 8
DELTA, FORGET, SSD = 0, 1, 2


def _lib():
    return kernels.lib(LIBRARY)


def _f32rows(t: torch.Tensor, what: str, n: int, cols: int) -> int:
    """Row stride of float32 rows [n, cols] (a column slice of a wider tensor is fine)."""
    if t.dtype != torch.float32 or t.dim() != 2 or t.stride(1) != 1 or tuple(t.shape) != (n, cols):
        raise ValueError(f"{what}: expected float32 rows [{n}, {cols}], got {tuple(t.shape)} {t.dtype} strides {t.stride()}")
    return t.stride(0)


def short_conv(u: torch.Tensor, weight: torch.Tensor, y: torch.Tensor, state: torch.Tensor, step, silu: bool,
               bias: Optional[torch.Tensor] = None, in_bias: Optional[torch.Tensor] = None) -> None:
    """y[t, c] = act(bias[c] + sum_j weight[c, j] * u[t - taps + 1 + j, c]) along each sequence, zeros before its
    start; ``state`` [slots, taps - 1, C] holds each sequence's last inputs and is advanced.  ``in_bias`` [C] is added
    to every input u[t, c] on the way in (not to the zeros before a sequence's start): the bias of the product
    that made the inputs, without a kernel of its own."""
    _dev(u, weight, y, state, bias, in_bias)
    _f32vec(bias, "conv bias", weight.shape[0])
    _f32vec(in_bias, "conv input bias", weight.shape[0])
    n = step.n_tokens
    c, taps = weight.shape
    ldu, ldy = _f32rows(u, "conv input", n, c), _f32rows(y, "conv output", n, c)
    if weight.dtype != torch.float32 or not weight.is_contiguous():
        raise TypeError("short_conv: the taps must be a contiguous float32 [channels, taps] tensor")
    if not 1 <= taps <= MAX_TAPS:
        raise ValueError(f"short_conv: {taps} taps (1 to {MAX_TAPS} are supported)")
    if state.dtype != torch.float32 or not state.is_contiguous() or tuple(state.shape[1:]) != (taps - 1, c):
        raise ValueError(f"short_conv: state must be float32 [slots, {taps - 1}, {c}], got {tuple(state.shape)}")
    if max(step.slots) >= state.shape[0]:
        raise ValueError("short_conv: a slot lies outside the state")
    library.call(_lib(), "agave_short_conv", ptr(u), ldu, ptr(weight), ptr(bias), ptr(y), ldy, ptr(state), ptr(step.tok_seq),
                 ptr(step.tok_pos), ptr(step.cu_dev), ptr(step.pos0_dev), ptr(step.slots_dev), n, step.n_seqs, c, taps,
                 1 if silu else 0, 1 if step.is_decode else 0, ptr(in_bias), stream())


def head_norm_rope_rows(q: Optional[torch.Tensor], k: Optional[torch.Tensor], v: Optional[torch.Tensor],
                        q_out: Optional[torch.Tensor], q_gain, k_gain, eps_q: float, eps_k: float,
                        freq: Optional[torch.Tensor], interleaved: bool, step, k_pages: Optional[torch.Tensor],
                        v_pages: Optional[torch.Tensor], table, base, n_heads: int, n_kv: int, dk: int, dv: int) -> None:
    """Per-head RMS norm (where a gain is given) and rotation of q and k; q to ``q_out`` (float32),
    k and v into their cache rows.  ``k`` None: only q (a run that appends nothing)."""
    _dev(q, k, v, q_out, q_gain, k_gain, freq, k_pages, v_pages, table, base)
    n = step.n_tokens
    ldq = ldqo = ldk = ldv = 0
    nh = nkv = width = n_pages = 0
    ref = None
    if q is not None:
        nh = n_heads
        ldq, ldqo = _f32rows(q, "q", n, nh * dk), _f32rows(q_out, "q_out", n, nh * dk)
        _f32vec(q_gain, "q_gain", dk)
    if k is not None:
        nkv = n_kv
        ldk, ldv = _f32rows(k, "k", n, nkv * dk), _f32rows(v, "v", n, nkv * dv)
        _f32vec(k_gain, "k_gain", dk)
        n_pages = check_row_pages(k_pages, v_pages, nkv, dk, dv)
        width = kernels._check_table(table, base, step.tok_seq)
        ref = k_pages
    rot_half = 0
    if freq is not None:
        if freq.dtype != torch.float64 or not freq.is_contiguous():
            raise TypeError("head_norm_rope_rows: frequencies are a contiguous float64 vector")
        rot_half = freq.numel()
        if 2 * rot_half > dk:
            raise ValueError(f"head_norm_rope_rows: {2 * rot_half} rotated elements exceed the head's {dk}")
    library.call(_lib(), "agave_head_norm_rope_rows", dt(ref) if ref is not None else kernels.F32, ptr(q), ldq, ptr(k), ldk,
                 ptr(v), ldv, ptr(q_out), ldqo, ptr(q_gain), ptr(k_gain), float(eps_q), float(eps_k),
                 1 if q_gain is not None else 0, 1 if k_gain is not None else 0, ptr(freq), rot_half,
                 1 if interleaved else 0, ptr(step.tok_seq), ptr(step.tok_pos), ptr(k_pages), ptr(v_pages), ptr(table),
                 width, ptr(base), n_pages, n, nh, nkv, dk, dv, stream())


def check_row_pages(k_pages: torch.Tensor, v_pages: torch.Tensor, nkv: int, dk: int, dv: int) -> int:
    if k_pages.dim() != 4 or tuple(k_pages.shape[1:]) != (nkv, 64, dk) or not k_pages.is_contiguous():
        raise ValueError(f"K pages must be contiguous [pages, {nkv}, 64, {dk}], got {tuple(k_pages.shape)}")
    if v_pages.dim() != 4 or tuple(v_pages.shape[1:]) != (nkv, 64, dv) or not v_pages.is_contiguous():
        raise ValueError(f"V pages must be contiguous [pages, {nkv}, 64, {dv}] (rows), got {tuple(v_pages.shape)}")
    if k_pages.shape[0] != v_pages.shape[0] or k_pages.dtype != v_pages.dtype:
        raise ValueError("K and V pages must agree in page count and dtype")
    return k_pages.shape[0]


def talk_attention(q: torch.Tensor, gate: Optional[torch.Tensor], out: torch.Tensor, k_pages: torch.Tensor,
                   v_pages: torch.Tensor, table, base, step, talk: Optional[torch.Tensor], n_heads: int, n_kv: int,
                   dk: int, dv: int, scale: float, chunk: Optional[int], out_scale: float = 1.0,
                   parts: Optional[torch.Tensor] = None) -> None:
    """Attention of every token over its sequence's cache rows, the heads' scores mixed by ``talk``
    [heads, heads] before the softmax; keys j <= p of the query's chunk (all if ``chunk`` is None);
    head h's output times sigmoid(gate[t, h]) (if given) and ``out_scale``, into ``out`` [N, heads * dv].
    ``parts`` (float32 [N, tiles, heads, dv + 2], with a chunk only, tiles * 64 >= chunk): a workgroup per
    token and tile of 64 keys leaves partial results there and a second kernel merges them, which is what
    a step of few tokens wants (one workgroup per token leaves the chip idle)."""
    _dev(q, gate, out, k_pages, v_pages, table, base, talk)
    n = step.n_tokens
    ldq = _f32rows(q, "q", n, n_heads * dk)
    ldg = _f32rows(gate, "gate", n, n_heads) if gate is not None else 0
    ldo = kernels._rows(out, "out")
    if tuple(out.shape) != (n, n_heads * dv) or out.dtype != k_pages.dtype:
        raise ValueError(f"talk_attention: out must be [{n}, {n_heads * dv}] of the cache's dtype")
    if talk is not None:
        _f32vec(talk.view(-1) if talk.is_contiguous() else talk, "talk", n_heads * n_heads)
    n_pages = check_row_pages(k_pages, v_pages, n_kv, dk, dv)
    width = kernels._check_table(table, base, step.tok_seq)
    if chunk is not None and chunk < 1:
        raise ValueError("talk_attention: a chunk holds at least one position")
    tiles = 0
    if parts is not None:
        _dev(parts)
        if chunk is None or parts.dtype != torch.float32 or not parts.is_contiguous() or parts.dim() != 4 \
                or tuple(parts.shape[0:1] + parts.shape[2:]) != (n, n_heads, dv + 2) or parts.shape[1] * 64 < chunk:
            raise ValueError(f"talk_attention: parts must be float32 [{n}, tiles, {n_heads}, {dv + 2}] with tiles * 64 >= chunk")
        tiles = parts.shape[1]
    library.call(_lib(), "agave_talk_attention", dt(out), ptr(q), ldq, ptr(gate), ldg, ptr(out), ldo, ptr(k_pages),
                 ptr(v_pages), ptr(table), width, ptr(base), n_pages, ptr(step.tok_seq), ptr(step.tok_pos), ptr(talk),
                 n, n_heads, n_kv, dk, dv, float(scale), int(chunk or 0), float(out_scale), ptr(parts), tiles, stream())


def gated_recurrence(mode: int, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, out: torch.Tensor,
                     state: torch.Tensor, step, n_heads: int, n_kv: int, dk: int, dv: int, *,
                     dt_in: Optional[torch.Tensor] = None, beta: Optional[torch.Tensor] = None,
                     a_log: Optional[torch.Tensor] = None, dt_bias: Optional[torch.Tensor] = None,
                     lower: Optional[torch.Tensor] = None, f_bias: Optional[torch.Tensor] = None,
                     skip: Optional[torch.Tensor] = None, unit_eps: float = 1e-6) -> None:
    """Advance ``state`` [slots, heads, dv, dk] (a column of S lies together) over the step's tokens, sequence by sequence, and
    write each token's read-out to ``out`` [N, heads * dv] (float32).

    ``DELTA``:  q, k [N, n_kv * dk] become unit vectors per head (q also times dk^-1/2);
    a = exp(-exp(a_log[h]) * softplus(dt_in + dt_bias)) per head and key channel; beta = sigmoid(beta);
    S <- diag(a) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q.
    ``FORGET``: q = silu(q), f = lower + (1 - lower) sigmoid(k + f_bias) with k the gate's input;
    S <- diag(f) S + (1 - f) v^T;  o = S^T q.
    ``SSD``:    q, k [N, n_kv * dk] as they come (head h reads group h // (heads / n_kv)); one step size per head
    and token, d = softplus(dt_in[t, h] + dt_bias[h]);  S <- exp(-exp(a_log[h]) d) S + d k v^T;  o = S^T q + skip[h] v."""
    _dev(q, k, v, out, state, dt_in, beta, a_log, dt_bias, lower, f_bias, skip)
    n = step.n_tokens
    kw = (n_heads if mode == FORGET else n_kv) * dk
    ldq, ldk = _f32rows(q, "q", n, kw), _f32rows(k, "k", n, kw)
    ldv, ldo = _f32rows(v, "v", n, n_heads * dv), _f32rows(out, "out", n, n_heads * dv)
    if state.dtype != torch.float32 or not state.is_contiguous() or tuple(state.shape[1:]) != (n_heads, dv, dk):
        raise ValueError(f"gated_recurrence: state must be float32 [slots, {n_heads}, {dv}, {dk}], got {tuple(state.shape)}")
    if max(step.slots) >= state.shape[0]:
        raise ValueError("gated_recurrence: a slot lies outside the state")
    lddt = ldb = 0
    if mode == DELTA:
        lddt, ldb = _f32rows(dt_in, "dt", n, n_heads * dk), _f32rows(beta, "beta", n, n_heads)
        _f32vec(a_log, "a_log", n_heads)
        _f32vec(dt_bias, "dt_bias", n_heads * dk)
        if a_log is None or dt_bias is None:
            raise ValueError("gated_recurrence: the delta rule needs a_log and dt_bias")
    elif mode == SSD:
        lddt = _f32rows(dt_in, "dt", n, n_heads)
        _f32vec(a_log, "a_log", n_heads)
        _f32vec(dt_bias, "dt_bias", n_heads)
        _f32vec(skip, "skip", n_heads)
        if a_log is None or dt_bias is None or skip is None:
            raise ValueError("gated_recurrence: the state-space form needs a_log, dt_bias and skip")
    elif mode == FORGET:
        _f32vec(lower, "lower", n_heads * dk)
        _f32vec(f_bias, "f_bias", n_heads * dk)
        if lower is None:
            raise ValueError("gated_recurrence: the forget gate needs its lower bound")
    else:
        raise ValueError(f"gated_recurrence: unknown mode {mode}")
    library.call(_lib(), "agave_gated_recurrence", mode, ptr(q), ldq, ptr(k), ldk, ptr(v), ldv, ptr(dt_in), lddt, ptr(beta),
                 ldb, ptr(a_log), ptr(dt_bias), ptr(lower), ptr(f_bias), ptr(skip), ptr(out), ldo, ptr(state), ptr(step.cu_dev),
                 ptr(step.slots_dev), step.n_seqs, n_heads, n_heads if mode == FORGET else n_kv, dk, dv, float(unit_eps),
                 1 if (step.is_decode and step.n_tokens == step.n_seqs) else 0, stream())


def head_norm_gate(o: torch.Tensor, weight: torch.Tensor, gate: Optional[torch.Tensor], out: torch.Tensor,
                   n_heads: int, dv: int, eps: float, out_scale: float = 1.0) -> None:
    """out[t, h] = o[t, h] / sqrt(mean(o[t, h]^2) + eps) * weight * sigmoid(gate[t, h]) * out_scale per head
    (``gate`` None: no gate); ``o`` and ``gate`` float32 [N, heads * dv], ``out`` in its own dtype."""
    _dev(o, weight, gate, out)
    n = o.shape[0]
    ldi = _f32rows(o, "o", n, n_heads * dv)
    ldg = _f32rows(gate, "gate", n, n_heads * dv) if gate is not None else 0
    ldo = kernels._rows(out, "out")
    if tuple(out.shape) != (n, n_heads * dv):
        raise ValueError(f"head_norm_gate: out must be [{n}, {n_heads * dv}], got {tuple(out.shape)}")
    _f32vec(weight, "weight", dv)
    library.call(_lib(), "agave_head_norm_gate", dt(out), ptr(o), ldi, ptr(weight), ptr(gate), ldg, ptr(out), ldo, n,
                 n_heads, dv, float(eps), float(out_scale), stream())


def gated_group_norm(y: torch.Tensor, z: torch.Tensor, weight: torch.Tensor, out: torch.Tensor, parts: int, eps: float) -> None:
    """g = y * silu(z); every one of the ``parts`` equal parts of a row of g is divided by its own root mean square
    (eps inside the root) and multiplied by ``weight`` [width]; ``y``, ``z`` float32 [N, width], ``out`` in its own dtype."""
    _dev(y, z, weight, out)
    n, width = y.shape
    if width % parts:
        raise ValueError(f"gated_group_norm: rows of {width} do not split into {parts} equal parts")
    ldy, ldz = _f32rows(y, "y", n, width), _f32rows(z, "z", n, width)
    ldo = kernels._rows(out, "out")
    if tuple(out.shape) != (n, width):
        raise ValueError(f"gated_group_norm: out must be [{n}, {width}], got {tuple(out.shape)}")
    _f32vec(weight, "weight", width)
    library.call(_lib(), "agave_gated_group_norm", dt(out), ptr(y), ldy, ptr(z), ldz, ptr(weight), ptr(out), ldo, n, parts,
                 width // parts, float(eps), stream())


def scaled_sum(a: torch.Tensor, sa: float, b: torch.Tensor, sb: float, out: torch.Tensor) -> None:
    """out = sa * a + sb * b, row by row (the three agree in shape and dtype)."""
    _dev(a, b, out)
    lda, ldb, ldo = kernels._rows(a, "a"), kernels._rows(b, "b"), kernels._rows(out, "out")
    if a.shape != b.shape or a.shape != out.shape or not (a.dtype == b.dtype == out.dtype):
        raise ValueError("scaled_sum: the three tensors must agree in shape and dtype")
    library.call(_lib(), "agave_scaled_sum", dt(out), ptr(a), lda, float(sa), ptr(b), ldb, float(sb), ptr(out), ldo,
                 a.shape[0], a.shape[1], stream())
