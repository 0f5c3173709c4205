"""Python faces of ``csrc/latent.hip``: the latents of the attention that caches one small row per position, and the
small products per (token, head) around its attention kernel.

Every function checks on the host what its kernel and grid assume and launches on the current stream.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import kernels, library
from .kernels import _P, _I, _L, _F, _dev, _f32vec, _i32, _rows, dt, ptr, stream

LIBRARY = "latent"

kernels.register_signatures(LIBRARY, {
    "agave_latent_prepare": [_I, _P, _L, _P, _P, _L, _I, _P, _L, _P, _P, _L, _I, _I, _P, _I, _P, _I, _F, _P],
    "agave_latent_expand": [_I, _P, _L, _P, _L, _P, _L, _I, _P, _L, _P, _I, _P, _I, _I, _I, _I, _P],
    "agave_gate_rows": [_I, _P, _L, _P, _L, _I, _I, _P],
    "agave_heads_product": [_I, _P, _L, _I, _P, _P, _L, _I, _P, _L, _P, _I, _I, _P, _I, _I, _I, _I, _I, _P],
})


def _lib():
    return kernels.lib(LIBRARY)


def _f32rows(t: torch.Tensor, what: str, n: int, cols: int) -> int:
    if t.dtype != torch.float32 or t.dim() != 2 or t.stride(1) != 1 or tuple(t.shape) != (n, cols):
        raise ValueError(f"{what}: expected float32 rows [{n}, {cols}], got {tuple(t.shape)} {t.dtype} strides {t.stride()}")
    return t.stride(0)


def latent_prepare(q_raw: torch.Tensor, q_weight: torch.Tensor, cq: torch.Tensor, kv_raw: Optional[torch.Tensor],
                   kv_weight: Optional[torch.Tensor], k_row: Optional[torch.Tensor], kv_rank: int, rot_dim: int,
                   freq: Optional[torch.Tensor], step, eps: float) -> None:
    """cq = q_raw / rms(q_raw) * q_weight; and, where ``kv_raw`` [N, kv_rank + rot_dim] is given,
    k_row = [kv_raw[:, :kv_rank] / rms(..) * kv_weight | the last rot_dim elements, the first 2 * len(freq) of them
    rotated in pairs (i, i + len(freq)) by position * freq[i]].  Raw rows are float32 (column slices are fine);
    ``cq`` and ``k_row`` have the activations' element type; eps stands inside the root."""
    _dev(q_raw, q_weight, cq, kv_raw, kv_weight, k_row, freq)
    n = step.n_tokens
    q_rank = q_raw.shape[1]
    ldq = _f32rows(q_raw, "query latent", n, q_rank)
    _f32vec(q_weight, "query latent's weight", q_rank)
    ldcq = _rows(cq, "cq")
    if tuple(cq.shape) != (n, q_rank):
        raise ValueError(f"latent_prepare: cq must be [{n}, {q_rank}], got {tuple(cq.shape)}")
    ldkv = ldkr = 0
    rot_half = 0
    if kv_raw is not None:
        ldkv = _f32rows(kv_raw, "key/value latent", n, kv_rank + rot_dim)
        _f32vec(kv_weight, "key/value latent's weight", kv_rank)
        ldkr = _rows(k_row, "k_row")
        if kv_weight is None or tuple(k_row.shape) != (n, kv_rank + rot_dim) or k_row.dtype != cq.dtype:
            raise ValueError(f"latent_prepare: k_row must be [{n}, {kv_rank + rot_dim}] of cq's dtype, with a weight")
        if freq is not None:
            rot_half = freq.numel()
            _f32vec(freq, "frequencies", rot_half)
            if 2 * rot_half > rot_dim:
                raise ValueError(f"latent_prepare: {2 * rot_half} rotated elements exceed the {rot_dim} there are")
        _i32(step.tok_pos, "positions", n)
    library.call(_lib(), "agave_latent_prepare", dt(cq), ptr(q_raw), ldq, ptr(q_weight), ptr(cq), ldcq, q_rank, ptr(kv_raw),
                 ldkv, ptr(kv_weight), ptr(k_row), ldkr, kv_rank, rot_dim, ptr(freq), rot_half, ptr(step.tok_pos), n,
                 float(eps), stream())


def heads_product(x: torch.Tensor, w: torch.Tensor, y: torch.Tensor, n_heads: int, x_head: int, y_head: int, *,
                  tail: int = 0, freq: Optional[torch.Tensor] = None, tok_pos: Optional[torch.Tensor] = None,
                  gate: Optional[torch.Tensor] = None, force_plain: bool = False) -> None:
    """For every token t and head h:  y[t, h * y_head + c] = sum_k w[h, c, k] * x[t, h * x_head + k]  (``w`` is
    [heads, n_out, K]); the head's next ``tail`` input elements are copied behind the product, the first
    2 * len(freq) of them rotated in pairs (i, i + len(freq)) by tok_pos[t] * freq[i]; with ``gate`` (float32
    [N, heads * n_out]) the product is multiplied by sigmoid(gate).  Sums are 32-bit; bfloat16 rows with K a multiple
    of 8 run on the matrix cores."""
    _dev(x, w, y, freq, tok_pos, gate)
    n = x.shape[0]
    ldx, ldy = _rows(x, "x"), _rows(y, "y")
    if w.dim() != 3 or w.shape[0] != n_heads or not w.is_contiguous() or w.dtype != x.dtype or y.dtype != x.dtype:
        raise ValueError(f"heads_product: w must be contiguous [{n_heads}, n_out, K] of the rows' dtype, and y of it too")
    n_out, k = int(w.shape[1]), int(w.shape[2])
    if y.shape[0] != n or x_head < k + tail or y_head < n_out + tail or x.shape[1] < (n_heads - 1) * x_head + k + tail \
            or y.shape[1] < (n_heads - 1) * y_head + n_out + tail:
        raise ValueError(f"heads_product: rows of {tuple(x.shape)} and {tuple(y.shape)} do not hold {n_heads} heads of "
                         f"{k} + {tail} in (every {x_head}) and {n_out} + {tail} out (every {y_head})")
    rot_half = 0
    if tail:
        if tok_pos is None:
            raise ValueError("heads_product: trailing elements need the tokens' positions")
        _i32(tok_pos, "positions", n)
        if freq is not None:
            rot_half = freq.numel()
            _f32vec(freq, "frequencies", rot_half)
            if 2 * rot_half > tail:
                raise ValueError(f"heads_product: {2 * rot_half} rotated elements exceed the {tail} trailing ones")
    ldg = 0
    if gate is not None:
        ldg = _f32rows(gate, "gate", n, n_heads * n_out)
    if (k + tail) * 4 > 64 * 1024:
        raise ValueError(f"heads_product: a head of {k + tail} input elements is too long")
    library.call(_lib(), "agave_heads_product", dt(x), ptr(x), ldx, x_head, ptr(w), ptr(y), ldy, y_head, ptr(gate), ldg,
                 ptr(freq), rot_half, tail, ptr(tok_pos), n, n_heads, n_out, k, 1 if force_plain else 0, stream())


def latent_expand(q: torch.Tensor, k_plain: torch.Tensor, k_row: torch.Tensor, kv_rank: int, k_full: torch.Tensor,
                  n_heads: int, dim: int, rot_dim: int, freq: Optional[torch.Tensor], tok_pos: torch.Tensor) -> None:
    """Every head's key row from the parts: k_full[t, h] = [k_plain[t, h] (``dim`` elements) | k_row[t, kv_rank:]
    (``rot_dim`` elements, rotated already)]; and the last ``rot_dim`` elements of every head of ``q``
    [N, heads * (dim + rot_dim)] are rotated in place (the first 2 * len(freq) of them, pairs (i, i + len(freq)), by
    tok_pos[t] * freq[i])."""
    _dev(q, k_plain, k_row, k_full, freq, tok_pos)
    n, qd = q.shape[0], dim + rot_dim
    ldq, ldkn, ldkr, ldkf = _rows(q, "q"), _rows(k_plain, "k_plain"), _rows(k_row, "k_row"), _rows(k_full, "k_full")
    if tuple(q.shape) != (n, n_heads * qd) or tuple(k_full.shape) != (n, n_heads * qd) or tuple(k_plain.shape) != (n, n_heads * dim) \
            or tuple(k_row.shape) != (n, kv_rank + rot_dim) or not (q.dtype == k_plain.dtype == k_row.dtype == k_full.dtype):
        raise ValueError(f"latent_expand: rows of {tuple(q.shape)}, {tuple(k_plain.shape)}, {tuple(k_row.shape)} and "
                         f"{tuple(k_full.shape)} do not hold {n_heads} heads of {dim} + {rot_dim} over a latent of {kv_rank}")
    _i32(tok_pos, "positions", n)
    rot_half = 0
    if freq is not None:
        rot_half = freq.numel()
        _f32vec(freq, "frequencies", rot_half)
        if 2 * rot_half > rot_dim:
            raise ValueError(f"latent_expand: {2 * rot_half} rotated elements exceed the {rot_dim} there are")
    library.call(_lib(), "agave_latent_expand", dt(q), ptr(q), ldq, ptr(k_plain), ldkn, ptr(k_row), ldkr, kv_rank, ptr(k_full),
                 ldkf, ptr(freq), rot_half, ptr(tok_pos), n, n_heads, dim, rot_dim, stream())


def gate_rows(x: torch.Tensor, gate: torch.Tensor) -> None:
    """x *= sigmoid(gate) in place; ``gate`` is float32 of ``x``'s shape (column slices are fine)."""
    _dev(x, gate)
    n, cols = x.shape
    ldx = _rows(x, "x")
    ldg = _f32rows(gate, "gate", n, cols)
    library.call(_lib(), "agave_gate_rows", dt(x), ptr(x), ldx, ptr(gate), ldg, n, cols, stream())
