"""Python faces of ``csrc/attention_biased.hip``: attention over cache pages stored row by row with a
bias on the scores that depends on the distance between query and key, a window with first
positions that stay visible, a sink in the softmax's denominator, and a gate on the output rows.

Every function checks on the host what its kernel and grid assume and launches on the current stream.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import kernels, library
from .kernels import _P, _I, _L, _F, _dev, _f32vec, _i32, _rows, dt, ptr, stream

LIBRARY = "attention_biased"

BIAS_NONE, BIAS_SLOPES, BIAS_TABLE = 0, 1, 2
MFMA_MAX_KEY, MFMA_MAX_VALUE = 576, 512         # the largest heads the matrix-core kernel takes
MAX_SPLITS = 16


def decode_splits(n_rows: int, n_kv: int, per: int, v_head_dim: int, table_width: int) -> int:
    """How many workgroups share the pages of one (row, key head) in a step of one row a sequence: enough to have some
    two hundred workgroups at work, never more than the longest sequence's pages give every wave one.  It depends on
    nothing that changes from step to step, so a recorded step stays valid."""
    waves = 8 if v_head_dim <= 128 else 4
    groups = max(1, n_rows * n_kv * ((per + 15) // 16))
    return max(1, min(MAX_SPLITS, 192 // groups, -(-table_width // waves)))

kernels.register_signatures(LIBRARY, {
    "agave_kv_append_rows": [_I, _P, _L, _P, _L, _P, _P, _P, _I, _P, _I, _I, _P, _P, _I, _I, _I, _I, _I, _P],
    "agave_attn_biased_plain": [_I, _P, _L, _P, _L, _P, _L, _P, _P, _P, _I, _P, _I, _I, _P, _P, _I, _I, _I, _I, _I, _F,
                                _I, _I, _I, _P, _I, _P, _I, _I, _F, _P],
    "agave_row_norm_rope": [_I, _P, _L, _P, _L, _P, _L, _P, _P, _P, _P, _L, _P, _L, _P, _L, _P, _P, _F, _F, _P, _I, _F, _P, _P,
                            _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _I, _I, _I, _P],
    "agave_attn_biased_mfma_ok": [_I, _I, _I, _I, _I],
    "agave_attn_biased_mfma": [_P, _L, _P, _L, _P, _L, _P, _P, _P, _I, _P, _I, _I, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I,
                               _F, _I, _I, _I, _P, _I, _P, _I, _P, _I, _F, _P],
})


def _lib():
    return kernels.lib(LIBRARY)


def _check_row_pages(k_pages: torch.Tensor, v_pages: torch.Tensor, nkv: int, hd: int, vd: int, dtype: torch.dtype,
                     packed: bool = False) -> int:
    if packed and (dtype != torch.bfloat16 or hd % 8 or vd % 16 or hd > MFMA_MAX_KEY or vd > MFMA_MAX_VALUE):
        raise ValueError(f"pages in operand order hold bfloat16, keys in steps of 8 up to {MFMA_MAX_KEY} and values in steps "
                         f"of 16 up to {MFMA_MAX_VALUE}")
    hd_k = (hd + 31) // 32 * 32 if packed else hd       # operands are whole steps of 32 along the head
    if k_pages.dim() != 4 or tuple(k_pages.shape[1:]) != (nkv, 64, hd_k) or not k_pages.is_contiguous():
        raise ValueError(f"K pages must be contiguous [pages, {nkv}, 64, {hd_k}], got {tuple(k_pages.shape)}")
    if v_pages.dim() != 4 or tuple(v_pages.shape[1:]) != (nkv, vd, 64) or not v_pages.is_contiguous():
        raise ValueError(f"V pages must be contiguous [pages, {nkv}, {vd}, 64], got {tuple(v_pages.shape)}")
    if k_pages.shape[0] != v_pages.shape[0] or k_pages.dtype != dtype or v_pages.dtype != dtype:
        raise ValueError("K and V pages must agree in page count and dtype with the activations")
    return k_pages.shape[0]


def _check_table(table: torch.Tensor, base: torch.Tensor, head: int, keep_first: int) -> int:
    width = kernels._check_table(table, base, None)
    if head < 0 or keep_first < 0 or keep_first > head * 64:
        raise ValueError(f"{keep_first} kept first positions need {-(-keep_first // 64)} kept pages, the table has {head}")
    return width


def kv_append_rows(k: torch.Tensor, v: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, table: torch.Tensor,
                   base: torch.Tensor, head: int, step, n_kv: int, head_dim: int, v_head_dim: int, packed: bool = False) -> None:
    """The step's key and value rows into their places in the cache pages: keys row by row and values transposed
    inside a page, or (``packed``) both in the order the matrix-core kernel reads its operands."""
    _dev(k, v, k_pages, v_pages, table, base)
    n = step.n_tokens
    ldk, ldv = _rows(k, "k"), _rows(v, "v")
    if k.shape != (n, n_kv * head_dim) or v.shape != (n, n_kv * v_head_dim) or k.dtype != v.dtype:
        raise ValueError(f"k and v must be [{n}, {n_kv * head_dim}] and [{n}, {n_kv * v_head_dim}] of one dtype")
    n_pages = _check_row_pages(k_pages, v_pages, n_kv, head_dim, v_head_dim, k.dtype, packed)
    width = _check_table(table, base, head, 0)
    library.call(_lib(), "agave_kv_append_rows", dt(k), ptr(k), ldk, ptr(v), ldv, ptr(k_pages), ptr(v_pages), ptr(table),
                 width, ptr(base), head, n_pages, ptr(step.tok_seq), ptr(step.tok_pos), n, n_kv, head_dim, v_head_dim,
                 1 if packed else 0, stream())


def attention(q: torch.Tensor, out: torch.Tensor, gate: Optional[torch.Tensor], k_pages: torch.Tensor,
              v_pages: torch.Tensor, table: torch.Tensor, base: torch.Tensor, head: int, step, n_heads: int, n_kv: int,
              head_dim: int, v_head_dim: int, scale: float, window: Optional[int], keep_first: int, bias_mode: int,
              bias: Optional[torch.Tensor], sink: Optional[torch.Tensor], packed: bool = False,
              force_plain: bool = False, workspace=None, splits: Optional[int] = None, chunk: Optional[int] = None,
              softcap: float = 0.0) -> None:
    """out[t, h] = sum_j w_j v_j with w = softmax_j(scale q.k_j + bias(h, p - j)) over the keys that token t at
    position p sees (j <= p and (p - j < window or j < keep_first)), the sink's exp(sink_h) added to the
    denominator, times sigmoid(gate[t, h]) element by element.  ``bias``: slopes [heads] (``BIAS_SLOPES``:
    the bias is -slope_h (p - j)) or a table [heads, distances] (``BIAS_TABLE``: distances beyond the table take
    its last column).  Pages in operand order (``packed``: bfloat16, a key size that is a multiple of 8 and a value size
    that is a multiple of 16, up to 576 and 512) run on the matrix cores, everything else (and everything with
    ``force_plain``) on the plain kernel, which reads either order.  With a ``workspace`` (something with
    ``get(name, rows, cols, dtype)``) a step of one row a sequence may share a row's pages among several workgroups,
    whose partial results a second kernel merges (``splits``: how many; None: :func:`decode_splits`).  ``chunk`` C: a
    token also sees only keys j with j // C == p // C.  ``softcap`` > 0: the scaled score becomes softcap * tanh(score /
    softcap) before the bias is added."""
    if chunk is not None and (chunk < 1 or keep_first):
        raise ValueError("attention: a chunk has at least one position and goes without kept first positions")
    if softcap < 0:
        raise ValueError("attention: a cap on the scores is positive (0: none)")
    _dev(q, out, gate, k_pages, v_pages, table, base, bias, sink)
    n = step.n_tokens
    ldq, ldo = _rows(q, "q"), _rows(out, "out")
    if q.shape != (n, n_heads * head_dim) or out.shape != (n, n_heads * v_head_dim) or out.dtype != q.dtype:
        raise ValueError(f"attention: q must be [{n}, {n_heads * head_dim}] and out [{n}, {n_heads * v_head_dim}] of one dtype")
    ldg = 0
    if gate is not None:
        ldg = _rows(gate, "gate")
        if gate.shape != out.shape or gate.dtype != q.dtype:
            raise ValueError("attention: the gate must have the output's shape and dtype")
    n_pages = _check_row_pages(k_pages, v_pages, n_kv, head_dim, v_head_dim, q.dtype, packed)
    width = _check_table(table, base, head, keep_first)
    bias_len = 0
    if bias_mode == BIAS_SLOPES:
        _f32vec(bias, "slopes", n_heads)
    elif bias_mode == BIAS_TABLE:
        if bias is None or bias.dtype != torch.float32 or bias.dim() != 2 or bias.shape[0] != n_heads or not bias.is_contiguous():
            raise ValueError(f"attention: the bias table must be contiguous float32 [{n_heads}, distances]")
        bias_len = bias.shape[1]
    elif bias_mode != BIAS_NONE:
        raise ValueError(f"attention: unknown bias mode {bias_mode}")
    _f32vec(sink, "sink", n_heads)
    if packed and not force_plain and _lib().agave_attn_biased_mfma_ok(head_dim, v_head_dim, ldq, ldo, ldg) \
            and q.data_ptr() % 16 == 0 and out.data_ptr() % 8 == 0:
        # the matrix cores: 16 rows of a head a wave in a step of many rows, a row's heads of one key head in a
        # step of one row a sequence
        _i32(step.cu_dev, "cu", step.n_seqs + 1)
        max_rows = max(b - a for a, b in zip(step.cu[:-1], step.cu[1:]))
        one_row = 1 if (step.is_decode and step.n_tokens == step.n_seqs) else 0
        parts = None
        if not one_row or workspace is None:
            splits = 1
        elif splits is None:
            splits = decode_splits(n, n_kv, n_heads // n_kv, v_head_dim, width)
        if not 1 <= splits <= 64:
            raise ValueError(f"attention: {splits} shares of a row (1 to 64)")
        if splits > 1:
            parts = workspace.get("attn_biased_parts", n * n_heads * splits, v_head_dim + 2, torch.float32)
        library.call(_lib(), "agave_attn_biased_mfma", ptr(q), ldq, ptr(out), ldo, ptr(gate), ldg, ptr(k_pages), ptr(v_pages),
                     ptr(table), width, ptr(base), head, n_pages, ptr(step.tok_seq), ptr(step.tok_pos), ptr(step.cu_dev), n,
                     step.n_seqs, max_rows, one_row, n_heads, n_kv, head_dim, v_head_dim, float(scale), int(window or 0),
                     int(keep_first), bias_mode, ptr(bias) if bias_mode != BIAS_NONE else None, bias_len, ptr(sink), splits,
                     ptr(parts), int(chunk or 0), float(softcap), stream())
        return
    library.call(_lib(), "agave_attn_biased_plain", dt(q), ptr(q), ldq, ptr(out), ldo, ptr(gate), ldg, ptr(k_pages),
                 ptr(v_pages), ptr(table), width, ptr(base), head, n_pages, ptr(step.tok_seq), ptr(step.tok_pos), n,
                 n_heads, n_kv, head_dim, v_head_dim, float(scale), int(window or 0), int(keep_first), bias_mode,
                 ptr(bias) if bias_mode != BIAS_NONE else None, bias_len, ptr(sink), 1 if packed else 0, int(chunk or 0),
                 float(softcap), stream())


def row_norm_rope(q: torch.Tensor, k: Optional[torch.Tensor], v: Optional[torch.Tensor], q_out: torch.Tensor,
                  k_out: Optional[torch.Tensor], v_out: Optional[torch.Tensor], q_weight: Optional[torch.Tensor],
                  k_weight: Optional[torch.Tensor], eps_q: float, eps_k: float, freq: Optional[torch.Tensor],
                  magnitude: float, step, n_heads: int, n_kv: int, head_dim: int, v_head_dim: int,
                  biases=(None, None, None), pages=None) -> None:
    """The 32-bit rows of a step's q, k and v (column slices are fine) into the rows the attention reads and the cache
    holds, in ``q_out``'s element type: ``biases`` (float32 vectors for q, k, v; any may be None) added; q and k divided
    by the root mean square of their whole row and multiplied by a weight per element (where a weight is given), then
    each head's first ``2 * len(freq)`` elements rotated, pair (e, e + len(freq)) by the angle ``pos * freq[e]`` (float64
    frequencies), sine and cosine times ``magnitude``; v converted.  ``k`` None: only q (a run that appends nothing).
    ``pages``: ``(k_pages, v_pages, table, base, kept pages, packed)``: the k and v rows go straight into their places in
    the cache (as :func:`kv_append_rows` would put them) and ``k_out`` / ``v_out`` are not used."""
    _dev(q, k, v, q_out, k_out, v_out, q_weight, k_weight, freq, *biases)
    n = step.n_tokens

    def f32rows(t, what, cols):
        if t.dtype != torch.float32 or t.dim() != 2 or t.stride(1) != 1 or tuple(t.shape) != (n, cols):
            raise ValueError(f"row_norm_rope: {what} must be float32 rows [{n}, {cols}], got {tuple(t.shape)} {t.dtype}")
        return t.stride(0)

    def outrows(t, what, cols):
        if t is None or t.dtype != q_out.dtype or t.dim() != 2 or t.stride(1) != 1 or tuple(t.shape) != (n, cols):
            raise ValueError(f"row_norm_rope: {what} must be rows [{n}, {cols}] of the result's dtype")
        return t.stride(0)
    qd, kd, vd = n_heads * head_dim, n_kv * head_dim, n_kv * v_head_dim
    ldq, ldqo = f32rows(q, "q", qd), outrows(q_out, "q_out", qd)
    ldk = ldv = ldko = ldvo = 0
    k_pages = v_pages = table = base = None
    head = width = n_pages = 0
    packed = False
    if k is not None:
        ldk, ldv = f32rows(k, "k", kd), f32rows(v, "v", vd)
        if pages is not None:
            k_pages, v_pages, table, base, head, packed = pages
            _dev(k_pages, v_pages, table, base)
            n_pages = _check_row_pages(k_pages, v_pages, n_kv, head_dim, v_head_dim, q_out.dtype, packed)
            width = _check_table(table, base, head, 0)
            k_out = v_out = None
        else:
            ldko, ldvo = outrows(k_out, "k_out", kd), outrows(v_out, "v_out", vd)
    _f32vec(q_weight, "q weight", qd)
    _f32vec(k_weight, "k weight", kd)
    for b, what, size in zip(biases, ("q bias", "k bias", "v bias"), (qd, kd, vd)):
        _f32vec(b, what, size)
    half = 0
    if freq is not None:
        if freq.dtype != torch.float64 or not freq.is_contiguous():
            raise TypeError("row_norm_rope: frequencies are a contiguous float64 vector")
        half = freq.numel()
        if 2 * half > head_dim or half > 256:
            raise ValueError(f"row_norm_rope: {2 * half} rotated elements in a head of {head_dim} (at most 512)")
    library.call(_lib(), "agave_row_norm_rope", dt(q_out), ptr(q), ldq, ptr(k), ldk, ptr(v), ldv, ptr(biases[0]), ptr(biases[1]),
                 ptr(biases[2]), ptr(q_out), ldqo, ptr(k_out), ldko, ptr(v_out), ldvo, ptr(q_weight), ptr(k_weight),
                 float(eps_q), float(eps_k), ptr(freq), half, float(magnitude), ptr(step.tok_pos),
                 ptr(step.tok_seq) if k_pages is not None else None,
                 ptr(k_pages), ptr(v_pages), ptr(table), width, ptr(base), int(head), n_pages, 1 if packed else 0,
                 n, n_heads, n_kv, head_dim, v_head_dim, stream())
