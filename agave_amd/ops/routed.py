"""Python faces of ``csrc/routed_ffn.hip``: the router's choice of experts and the experts' products."""
from __future__ import annotations

from typing import Optional

import torch

from . import kernels, library
from .kernels import _P, _I, _L, _F, _dev, _f32vec, _i32, _rows, dt, ptr, stream

LIBRARY = "routed_ffn"
MAX_OUTPUTS = 1024

kernels.register_signatures(LIBRARY, {
    "agave_route_topk": [_P, _L, _P, _P, _I, _I, _I, _I, _I, _F, _P, _P, _P],
    "agave_routed_experts_plain": [_I, _P, _L, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _F, _P],
    "agave_route_rows": [_I, _P, _L, _P, _P, _I, _I, _I, _I, _I, _I, _F, _P, _P, _I, _I, _P, _I, _I, _P],
    "agave_route_sort": [_P, _I, _I, _I, _I, _I, _P, _P, _P, _P],
    "agave_routed_experts_mfma": [_P, _L, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _F, _F, _P],
    "agave_routed_combine": [_I, _P, _P, _P, _P, _P, _L, _P, _L, _P, _P, _L, _I, _I, _I, _I, _P],
})


def _lib():
    return kernels.lib(LIBRARY)


def route_topk(logits: torch.Tensor, correction: Optional[torch.Tensor], scratch: torch.Tensor, groups: int, keep: int,
               top: int, scale: float, choice: torch.Tensor, weight: torch.Tensor) -> None:
    """For every row of 32-bit router logits [N, R]: s = softmax; among the outputs of the ``keep`` groups (of
    ``groups`` equal groups of neighbours) whose largest ``s + correction`` is largest, the ``top`` outputs with the
    largest ``s + correction`` go to ``choice`` [N, top] (int32) and ``s * scale`` to ``weight`` [N, top]."""
    _dev(logits, correction, scratch, choice, weight)
    n, r = logits.shape
    if logits.dtype != torch.float32 or logits.stride(1) != 1:
        raise TypeError("route_topk: router logits must be float32 rows")
    _f32vec(correction, "correction", r)
    if scratch.dtype != torch.float32 or not scratch.is_contiguous() or scratch.numel() < n * r:
        raise ValueError("route_topk: scratch must hold a float32 value per logit")
    _i32(choice, "choice", n * top)
    if weight.dtype != torch.float32 or not weight.is_contiguous() or weight.numel() < n * top:
        raise ValueError("route_topk: weight must be contiguous float32 [N, top]")
    library.call(_lib(), "agave_route_topk", ptr(logits), logits.stride(0), ptr(correction), ptr(scratch), n, r, groups, keep,
                 top, float(scale), ptr(choice), ptr(weight), stream())


def experts_plain(x: torch.Tensor, choice: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor,
                  act_rows: torch.Tensor, y: torch.Tensor, top: int, activation: int, p0: float = 0.0, p1: float = 1.0) -> None:
    """y[p] = W_down[e] (act(W_gate[e] x_t) * (W_up[e] x_t)) for every pair p = t * top + slot whose choice e is an
    expert with weights (e < E); rows of other pairs are left alone.  ``y`` is float32 [N * top, hidden]."""
    _dev(x, choice, w_gate, w_up, w_down, act_rows, y)
    n, hidden = x.shape
    ldx = _rows(x, "x")
    e, ff, k = w_gate.shape
    if k != hidden or w_up.shape != w_gate.shape or w_down.shape != (e, hidden, ff):
        raise ValueError("experts: weights must be [E, ff, hidden], [E, ff, hidden] and [E, hidden, ff]")
    for w in (w_gate, w_up, w_down):
        if w.dtype != x.dtype or not w.is_contiguous():
            raise TypeError("experts: weights must be contiguous and of the rows' dtype")
    _i32(choice, "choice", n * top)
    if act_rows.dtype != x.dtype or not act_rows.is_contiguous() or act_rows.shape != (n * top, ff):
        raise ValueError(f"experts: inner rows must be [{n * top}, {ff}] of the rows' dtype")
    if y.dtype != torch.float32 or not y.is_contiguous() or y.shape != (n * top, hidden):
        raise ValueError(f"experts: y must be float32 [{n * top}, {hidden}]")
    library.call(_lib(), "agave_routed_experts_plain", dt(x), ptr(x), ldx, ptr(choice), ptr(w_gate), ptr(w_up), ptr(w_down),
                 ptr(act_rows), ptr(y), n, top, e, ff, hidden, activation, float(p0), float(p1), stream())


def combine(y: Optional[torch.Tensor], place: Optional[torch.Tensor], choice: torch.Tensor, weight: torch.Tensor,
            x: torch.Tensor, shared: Optional[torch.Tensor], out: torch.Tensor, top: int, n_experts: int,
            shared_gate: Optional[torch.Tensor] = None) -> None:
    """out[t] = sum over the token's pairs of weight * (the pair's expert row of ``y``, or ``x[t]`` itself where the
    choice is an identity expert, e >= n_experts) + shared[t], the latter times ``sigmoid(shared_gate[t])`` where a
    float32 logit per token is given."""
    _dev(y, place, choice, weight, x, shared, out, shared_gate)
    _f32vec(shared_gate, "shared_gate", x.shape[0])
    n, hidden = x.shape
    ldx, ldo = _rows(x, "x"), _rows(out, "out")
    if out.shape != x.shape or out.dtype != x.dtype:
        raise ValueError("combine: out must have the input's shape and dtype")
    lds = 0
    if shared is not None:
        lds = _rows(shared, "shared")
        if shared.shape != x.shape or shared.dtype != x.dtype:
            raise ValueError("combine: the shared expert's rows must have the input's shape and dtype")
    if y is not None and (y.dtype != torch.float32 or not y.is_contiguous() or y.shape[1] != hidden or y.shape[0] < n * top):
        raise ValueError("combine: y must be float32 [>= N * top, hidden]")
    _i32(choice, "choice", n * top)
    _i32(place, "place", n * top)
    library.call(_lib(), "agave_routed_combine", dt(x), ptr(y), ptr(place), ptr(choice), ptr(weight), ptr(x), ldx, ptr(shared),
                 lds, ptr(shared_gate) if shared is not None else None, ptr(out), ldo, n, top, n_experts, hidden, stream())


def tile_plan(n_pairs: int, n_experts: int):
    """(rows a tile, tiles at most, sorted rows at most) of the sorted list of ``n_pairs`` pairs: tiles of 64 rows
    where an expert gets some 32 pairs or more on average, of 16 otherwise; every expert's run of rows is padded to
    whole tiles, so there are at most ``ceil(pairs / rows) + experts`` tiles."""
    tm = 64 if n_pairs >= 32 * n_experts else 16
    tiles = (n_pairs + tm - 1) // tm + n_experts
    return tm, tiles, tiles * tm


def mfma_ok(x: torch.Tensor, ff: int) -> bool:
    """Whether the matrix-core kernels take these rows (bfloat16, sizes that are multiples of 8, aligned)."""
    return (x.dtype == torch.bfloat16 and x.shape[1] % 8 == 0 and ff % 8 == 0 and x.stride(0) % 8 == 0
            and x.data_ptr() % 16 == 0)


def route_sort(choice: torch.Tensor, n_experts: int, tm: int, tiles: int, place: torch.Tensor, sorted_pair: torch.Tensor,
               tile_expert: torch.Tensor) -> None:
    """Sort the pairs by expert on the device: ``place[p]`` the sorted row of pair p (-1 for an identity expert),
    ``sorted_pair[r]`` the pair in sorted row r (-1: padding), ``tile_expert[t]`` the expert of tile t (-1: none)."""
    _dev(choice, place, sorted_pair, tile_expert)
    p = choice.numel()
    _i32(choice, "choice")
    _i32(place, "place", p)
    _i32(sorted_pair, "sorted_pair", tiles * tm)
    _i32(tile_expert, "tile_expert", tiles)
    library.call(_lib(), "agave_route_sort", ptr(choice), p, n_experts, tm, tiles * tm, tiles, ptr(place), ptr(sorted_pair),
                 ptr(tile_expert), stream())


def experts_mfma(x: torch.Tensor, sorted_pair: torch.Tensor, tile_expert: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor,
                 w_down: torch.Tensor, act_rows: torch.Tensor, y: torch.Tensor, tm: int, tiles: int, top: int, activation: int,
                 tile_order: bool = False, p0: float = 0.0, p1: float = 1.0) -> None:
    """The experts' products over the sorted rows on the matrix cores: ``act_rows`` [tiles * tm, ff] bfloat16 and
    ``y`` [tiles * tm, hidden] float32 receive sorted rows (padding rows hold nothing of use).  ``tile_order``: the
    weights were rearranged by :func:`pack_expert_weights` (same shapes)."""
    _dev(x, sorted_pair, tile_expert, w_gate, w_up, w_down, act_rows, y)
    n, hidden = x.shape
    e, ff, k = w_gate.shape
    if k != hidden or w_up.shape != w_gate.shape or w_down.shape != (e, hidden, ff):
        raise ValueError("experts: weights must be [E, ff, hidden], [E, ff, hidden] and [E, hidden, ff]")
    for w in (w_gate, w_up, w_down):
        if w.dtype != torch.bfloat16 or not w.is_contiguous():
            raise TypeError("experts: the matrix-core kernels take contiguous bfloat16 weights")
    if not mfma_ok(x, ff):
        raise ValueError("experts: rows that the matrix-core kernels do not take")
    cap = tiles * tm
    if act_rows.dtype != torch.bfloat16 or not act_rows.is_contiguous() or act_rows.shape != (cap, ff):
        raise ValueError(f"experts: inner rows must be bfloat16 [{cap}, {ff}]")
    if y.dtype != torch.float32 or not y.is_contiguous() or y.shape != (cap, hidden):
        raise ValueError(f"experts: y must be float32 [{cap}, {hidden}]")
    _i32(sorted_pair, "sorted_pair", cap)
    _i32(tile_expert, "tile_expert", tiles)
    library.call(_lib(), "agave_routed_experts_mfma", ptr(x), x.stride(0), ptr(sorted_pair), ptr(tile_expert), ptr(w_gate),
                 ptr(w_up), ptr(w_down), ptr(act_rows), ptr(y), tm, tiles, top, e, ff, hidden, activation,
                 1 if tile_order else 0, float(p0), float(p1), stream())


def route_rows(x: torch.Tensor, router: torch.Tensor, correction: Optional[torch.Tensor], groups: int, keep: int, top: int,
               scale: float, choice: torch.Tensor, weight: torch.Tensor, softmax_top: bool = False,
               extra_out: Optional[torch.Tensor] = None, sigmoid: bool = False, group_top: int = 1,
               normalise: bool = False) -> None:
    """The router's 32-bit product ``x router^T`` and :func:`route_topk`'s choice in one kernel (the logits never
    leave the compute unit).  ``router`` is float32 [R, width]; ``x`` [N, width] in either element type.
    ``softmax_top``: the ``top`` largest logits + ``correction`` are chosen (the lower index among equals) and their
    weights are the softmax over the chosen alone, times ``scale`` (no groups, ``top`` <= 64).  ``extra_out``
    (float32 [N, extra]): the router matrix has ``extra`` further rows behind its outputs, whose products with
    the rows are left there as they are.  ``sigmoid``: the scores are the logits' sigmoids instead of their softmax.
    ``group_top`` 2: a group counts by the sum of its two largest scores + correction.  ``normalise``: the chosen
    weights are divided by their sum + 1e-20 before ``scale`` (``top`` <= 64)."""
    _dev(x, router, correction, choice, weight, extra_out)
    n, k = x.shape
    ldx = _rows(x, "x")
    if router.dtype != torch.float32 or router.dim() != 2 or router.shape[1] != k or not router.is_contiguous():
        raise ValueError(f"route_rows: the router must be contiguous float32 [outputs, {k}]")
    extra = 0
    if extra_out is not None:
        if extra_out.dtype != torch.float32 or extra_out.dim() != 2 or extra_out.shape[0] != n or not extra_out.is_contiguous():
            raise ValueError(f"route_rows: extra_out must be contiguous float32 [{n}, extra]")
        extra = extra_out.shape[1]
    r = router.shape[0] - extra
    if r < 1:
        raise ValueError("route_rows: the router has no outputs")
    if softmax_top and (groups != 1 or keep != 1 or top > 64):
        raise ValueError("route_rows: the softmax over the chosen logits takes no groups and at most 64 chosen")
    if softmax_top and (sigmoid or normalise):
        raise ValueError("route_rows: one way of scoring at a time")
    if group_top not in (1, 2) or (normalise and top > 64):
        raise ValueError("route_rows: a group counts by its largest or its two largest scores; weights are divided by their "
                         "sum for at most 64 chosen")
    _f32vec(correction, "correction", r)
    _i32(choice, "choice", n * top)
    if weight.dtype != torch.float32 or not weight.is_contiguous() or weight.numel() < n * top:
        raise ValueError("route_rows: weight must be contiguous float32 [N, top]")
    library.call(_lib(), "agave_route_rows", dt(x), ptr(x), ldx, ptr(router), ptr(correction), n, k, r, groups, keep, top,
                 float(scale), ptr(choice), ptr(weight), 1 if softmax_top else (2 if sigmoid else 0), extra, ptr(extra_out),
                 int(group_top), 1 if normalise else 0, stream())


def pack_expert_weights(w: torch.Tensor) -> torch.Tensor:
    """[E, N, K] (N a multiple of 16, K of 32) rearranged into the matrix cores' operand tiles: tiles of 16 rows by 32
    columns, each stored as its 64 lanes' 16 bytes one after another (lane c + 16 g holds row c, columns 8 g .. 8 g + 7),
    a row block's tiles along K following each other.  Same shape and bytes; only :func:`experts_mfma` reads it."""
    e, n, k = w.shape
    if n % 16 or k % 32:
        raise ValueError("pack_expert_weights: rows must be a multiple of 16 and columns of 32")
    t = w.view(e, n // 16, 16, k // 32, 4, 8).permute(0, 1, 3, 4, 2, 5).contiguous()      # [E, nb, kb, g, c, 8]
    return t.view(e, n, k)
