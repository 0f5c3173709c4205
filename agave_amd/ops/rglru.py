"""Python faces of ``csrc/rglru.hip``: the gates and the scan of a gated linear recurrence per channel."""
from __future__ import annotations

import torch

from . import kernels, library
from .kernels import _P, _I, _L, _dev, _f32vec, dt, ptr, stream
from .sequence import _f32rows

LIBRARY = "rglru"
CHUNK = 32                     # rows of a step that one thread walks through in the scan

kernels.register_signatures(LIBRARY, {
    "agave_rglru_gates": [_I, _P, _L, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _P],
    "agave_rglru_scan": [_P, _P, _P, _L, _P, _P, _I, _L, _P, _P, _P, _P, _P, _L, _I, _I, _I, _I, _I, _P],
})


def _lib():
    return kernels.lib(LIBRARY)


def gates(u: torch.Tensor, w_r: torch.Tensor, w_i: torch.Tensor, b_r: torch.Tensor, b_i: torch.Tensor, decay: torch.Tensor,
          a_out: torch.Tensor, x_out: torch.Tensor) -> None:
    """In every block b of channels: ``r = sigmoid(w_r[b] u_b + b_r[b])``, ``g = sigmoid(w_i[b] u_b + b_i[b])``;
    ``a_out = exp(-decay r)``, ``x_out = sqrt(1 - a^2) g u``.  ``u`` float32 [N, W] (a column slice is fine); the gate
    matrices [blocks, W / blocks, W / blocks] in either element type; everything else float32."""
    _dev(u, w_r, w_i, b_r, b_i, decay, a_out, x_out)
    n, w = u.shape
    ldu = _f32rows(u, "rglru input", n, w)
    blocks = w_r.shape[0]
    if w % blocks or tuple(w_r.shape) != (blocks, w // blocks, w // blocks) or w_i.shape != w_r.shape \
            or w_i.dtype != w_r.dtype or not w_r.is_contiguous() or not w_i.is_contiguous():
        raise ValueError(f"rglru.gates: gate matrices must be contiguous [blocks, {w} / blocks, {w} / blocks] of one dtype")
    for t, what in ((b_r, "r bias"), (b_i, "i bias"), (decay, "decay")):
        if t is None or t.dtype != torch.float32 or not t.is_contiguous() or t.numel() != w:
            raise TypeError(f"rglru.gates: {what} must hold {w} contiguous float32 values")
    for t in (a_out, x_out):
        if t.dtype != torch.float32 or not t.is_contiguous() or tuple(t.shape) != (n, w):
            raise ValueError(f"rglru.gates: results must be contiguous float32 [{n}, {w}]")
    library.call(_lib(), "agave_rglru_gates", dt(w_r), ptr(u), ldu, ptr(w_r), ptr(w_i), ptr(b_r), ptr(b_i), ptr(decay),
                 ptr(a_out), ptr(x_out), n, w, blocks, stream())


def scan(a: torch.Tensor, x: torch.Tensor, y: torch.Tensor, out: torch.Tensor, state: torch.Tensor, step, workspace,
         y_bias=None) -> None:
    """``S_t = a_t S_(t-1) + x_t`` along every sequence of the step, from the sequence's ``state`` [slots, W], which is
    left at the last row's; ``out_t = S_t gelu_tanh(y_t + y_bias)``.  ``a``, ``x`` contiguous float32 [N, W]; ``y`` float32
    rows; ``y_bias`` float32 [W] or None."""
    _dev(a, x, y, out, state, y_bias)
    _f32vec(y_bias, "y bias", a.shape[1])
    n, w = a.shape
    if n != step.n_tokens:
        raise ValueError("rglru.scan: a row per token of the step")
    for t in (a, x):
        if t.dtype != torch.float32 or not t.is_contiguous() or tuple(t.shape) != (n, w):
            raise ValueError(f"rglru.scan: a and x must be contiguous float32 [{n}, {w}]")
    ldy = _f32rows(y, "rglru y", n, w)
    if out.dim() != 2 or tuple(out.shape) != (n, w) or out.stride(1) != 1:
        raise ValueError(f"rglru.scan: out must be [{n}, {w}]")
    if state.dtype != torch.float32 or not state.is_contiguous() or state.dim() != 2 or state.shape[1] != w:
        raise ValueError(f"rglru.scan: state must be contiguous float32 [slots, {w}]")
    if max(step.slots) >= state.shape[0]:
        raise ValueError("rglru.scan: a slot lies outside the state")
    # a step of one row a sequence (every decode step): the rows do not depend on each other
    one_each = bool(step.is_decode and n == step.n_seqs)
    chunks = (n + CHUNK - 1) // CHUNK
    scratch, floats = None, 0
    if chunks > 1 and not one_each:
        floats = (3 * chunks + step.n_seqs) * w
        scratch = workspace.get("rglru_scan_scratch", 3 * chunks + step.n_seqs, w, torch.float32)
    library.call(_lib(), "agave_rglru_scan", ptr(a), ptr(x), ptr(y), ldy, ptr(y_bias), ptr(out), dt(out), out.stride(0), ptr(state),
                 ptr(step.tok_seq), ptr(step.cu_dev), ptr(step.slots_dev), ptr(scratch), floats, n, step.n_seqs, w, CHUNK,
                 1 if one_each else 0, stream())
