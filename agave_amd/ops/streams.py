"""Python faces of ``csrc/streams.hip``: several residual streams per token."""
from __future__ import annotations

from typing import Optional

import torch

from . import kernels, library
from .kernels import _P, _I, _L, _F, _dev, _f32vec, _i32, dt, ptr, stream

LIBRARY = "streams"
MAX_STREAMS, MAX_WIDTH = 16, 15360
NORM_NONE, NORM_LAYER, NORM_RMS = 0, 1, 2

kernels.register_signatures(LIBRARY, {
    "agave_streams_step": [_P, _I, _I, _I, _P, _I, _L, _I, _L, _P, _P, _P, _I, _P, _P, _F, _P, _I, _L, _P, _I, _P],
    "agave_streams_fill": [_P, _P, _I, _I, _I, _P],
})


def _lib():
    return kernels.lib(LIBRARY)


def _check_streams(h: torch.Tensor, streams: int, width: int) -> int:
    if h.dtype != torch.float32 or h.dim() != 2 or h.shape[1] != streams * width or not h.is_contiguous():
        raise ValueError(f"streams: the residual must be contiguous float32 [tokens, {streams} * {width}], got {tuple(h.shape)} {h.dtype}")
    if not 1 <= streams <= MAX_STREAMS or not 1 <= width <= MAX_WIDTH:
        raise ValueError(f"streams: {streams} streams of {width} elements (1 to {MAX_STREAMS} streams, up to {MAX_WIDTH} elements)")
    return h.shape[0]


def fill(x: torch.Tensor, h: torch.Tensor, streams: int) -> None:
    """h[t, s, :] = x[t, :] for every stream s: all streams start as the token's row."""
    _dev(x, h)
    n = _check_streams(h, streams, x.shape[1])
    if x.dtype != torch.float32 or not x.is_contiguous() or x.shape[0] != n:
        raise ValueError("streams.fill: the rows must be contiguous float32 [tokens, width]")
    library.call(_lib(), "agave_streams_fill", ptr(x), ptr(h), n, streams, x.shape[1], stream())


def step(h: torch.Tensor, streams: int, width: int, branch: Optional[torch.Tensor], mix: Optional[torch.Tensor],
         write: Optional[torch.Tensor], read: Optional[torch.Tensor], norm_kind: int, weight: Optional[torch.Tensor],
         bias: Optional[torch.Tensor], eps: float, out: Optional[torch.Tensor], rows: Optional[torch.Tensor] = None) -> None:
    """With a ``branch`` y ([tokens, width] in either element type, or float32 slices [slices, tokens, width] that add up
    to it): ``x_t <- sum_s mix[s, t] x_s + write[t] y`` for all streams t at once.  With ``out``: ``out = norm(sum_s
    read[s] x_s)`` of the streams as they then are (layer norm with weight and optional bias, RMS norm with weight, or
    none).  ``rows`` (int32): only these tokens are visited, ``out`` has a row for each, and no stream is stored."""
    _dev(h, branch, mix, write, read, weight, bias, out, rows)
    n = _check_streams(h, streams, width)
    y_dt, ldy, slices, slice_stride = 0, 0, 1, 0
    if branch is not None:
        if branch.dim() == 3:
            if branch.dtype != torch.float32 or branch.shape[1:] != (n, width) or branch.stride(2) != 1:
                raise ValueError("streams.step: slices must be float32 [slices, tokens, width]")
            slices, slice_stride, ldy = branch.shape[0], branch.stride(0), branch.stride(1)
        else:
            if branch.dim() != 2 or tuple(branch.shape) != (n, width) or branch.stride(1) != 1:
                raise ValueError(f"streams.step: the branch must be [{n}, {width}], got {tuple(branch.shape)}")
            ldy = branch.stride(0)
        y_dt = dt(branch)
        _f32vec(write, "write", streams)
        if mix is None or mix.dtype != torch.float32 or not mix.is_contiguous() or tuple(mix.shape) != (streams, streams):
            raise ValueError(f"streams.step: mix must be contiguous float32 [{streams}, {streams}]")
        if write is None:
            raise ValueError("streams.step: a branch needs the coefficients it is written with")
    o_dt, ldo, n_rows = 0, 0, 0
    if out is not None:
        _f32vec(read, "read", streams)
        if read is None:
            raise ValueError("streams.step: rows to hand on need the coefficients they are read with")
        n_out = n if rows is None else rows.numel()
        if out.dim() != 2 or tuple(out.shape) != (n_out, width) or out.stride(1) != 1:
            raise ValueError(f"streams.step: out must be [{n_out}, {width}], got {tuple(out.shape)}")
        o_dt, ldo = dt(out), out.stride(0)
        if norm_kind != NORM_NONE:
            _f32vec(weight, "norm weight", width)
            _f32vec(bias, "norm bias", width)
            if weight is None:
                raise ValueError("streams.step: a norm needs its weight")
    elif rows is not None:
        raise ValueError("streams.step: chosen rows are for handing rows on")
    if rows is not None:
        _i32(rows, "rows")
        n_rows = rows.numel()
    library.call(_lib(), "agave_streams_step", ptr(h), n, streams, width, ptr(branch), y_dt, ldy, slices, slice_stride,
                 ptr(mix), ptr(write), ptr(read) if out is not None else None, int(norm_kind), ptr(weight), ptr(bias),
                 float(eps), ptr(out), o_dt, ldo, ptr(rows), n_rows, stream())
