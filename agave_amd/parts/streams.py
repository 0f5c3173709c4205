"""Several residual streams per token (hyper-connections): the block arrangement ``streams``.

The residual of a token is S rows ``x_1 .. x_S`` (``ModelSpec.streams``), all equal to the embedding row at the start.
Sublayer q of a layer has three small tensors: it reads ``u = sum_s read[s] x_s``, runs ``y = f(norm(u))``, and writes, for
every stream t at once from the old rows,

    x_t <- sum_s mix[s, t] x_s + write[t] y

The model's end takes the streams' sum through the final norm.  As with one residual, a block never writes its last
result itself: it returns it as *pending* ``(y, StreamMix)``, and the kernel that reads the streams for the next sublayer
(or for the model's end) writes it first, so the streams are read and written once per sublayer.
"""
from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from ..config.spec import LayerSpec, StreamMixSpec
from ..ops import streams as ops
from ..weights.loader import TensorNeed
from .base import BuildEnv, lookup, register
from .norm import LayerNorm, RmsNorm


class StreamMix:
    """One sublayer's coefficients on the device, in 32-bit."""

    def __init__(self, spec: StreamMixSpec, weights, env: BuildEnv):
        def vec(name, shape):
            t = weights.get(name).to(torch.float32)
            if tuple(t.shape) != shape:
                raise ValueError(f"{name}: expected shape {shape}, got {tuple(t.shape)}")
            return t.contiguous().to(env.device)
        s = spec.streams
        self.streams = s
        self.read, self.write, self.mix = vec(spec.read, (s,)), vec(spec.write, (s,)), vec(spec.mix, (s, s))

    @staticmethod
    def tensor_needs(spec: StreamMixSpec) -> List[TensorNeed]:
        s = spec.streams
        return [TensorNeed(spec.read, (s,), init="mean"), TensorNeed(spec.write, (s,), init="ones"),
                TensorNeed(spec.mix, (s, s), init="identity")]


def _norm_arguments(norm):
    if norm is None:
        return ops.NORM_NONE, None, None, 0.0
    if isinstance(norm, LayerNorm):
        return ops.NORM_LAYER, norm.weight, norm.bias, norm.eps
    if isinstance(norm, RmsNorm):
        return ops.NORM_RMS, norm.gain, None, norm.eps
    raise ValueError(f"a block of several streams takes a layer norm or an RMS norm in front of a sublayer, got {type(norm).__name__}")


def write_and_read(h: torch.Tensor, streams: int, width: int, pending, read: Optional[torch.Tensor], norm,
                   out: Optional[torch.Tensor], rows: Optional[torch.Tensor] = None) -> None:
    """Write the pending result into the streams ``h`` [tokens, streams * width], then ``out = norm(sum_s read[s] x_s)``
    (of the chosen rows only, storing nothing, if ``rows`` is given)."""
    branch, how = pending if pending is not None else (None, None)
    kind, w, b, eps = _norm_arguments(norm)
    if rows is not None and branch is not None and out is None:
        raise ValueError("chosen rows are for handing rows on")
    ops.step(h, streams, width, branch, how.mix if how is not None else None, how.write if how is not None else None,
             read, kind, w, b, eps, out, rows)


class StreamsBlock:
    def __init__(self, spec: LayerSpec, weights, env: BuildEnv):
        self.spec, self.env = spec, env

        def norm(ns):
            return lookup("norm", ns.kind)(ns, weights, env) if ns is not None else None
        if spec.post_mixer_norm is not None or spec.post_ffn_norm is not None:
            raise ValueError("a block of several streams has no norm behind a sublayer")
        if spec.mixer_streams is None or (spec.ffn is not None and spec.ffn_streams is None):
            raise ValueError("a block of several streams needs every sublayer's coefficients")
        self.pre_mixer, self.pre_ffn = norm(spec.pre_mixer_norm), norm(spec.pre_ffn_norm)
        _norm_arguments(self.pre_mixer), _norm_arguments(self.pre_ffn)
        self.mixer_streams = StreamMix(spec.mixer_streams, weights, env)
        self.ffn_streams = StreamMix(spec.ffn_streams, weights, env) if spec.ffn is not None else None
        self.streams = spec.mixer_streams.streams
        if self.ffn_streams is not None and self.ffn_streams.streams != self.streams:
            raise ValueError("a layer's sublayers must agree in the number of streams")
        self.mixer = lookup("mixer", spec.mixer.kind)(spec.mixer, weights, env)
        self.ffn = lookup("ffn", spec.ffn.kind)(spec.ffn, weights, env) if spec.ffn is not None else None
        self.hidden = spec.mixer.hidden

    @classmethod
    def tensor_needs(cls, spec: LayerSpec) -> List[TensorNeed]:
        needs: List[TensorNeed] = []
        for ns in (spec.pre_mixer_norm, spec.pre_ffn_norm):
            if ns is not None:
                needs += lookup("norm", ns.kind).tensor_needs(ns)
        for ss in (spec.mixer_streams, spec.ffn_streams):
            if ss is not None:
                needs += StreamMix.tensor_needs(ss)
        needs += lookup("mixer", spec.mixer.kind).tensor_needs(spec.mixer)
        if spec.ffn is not None:
            needs += lookup("ffn", spec.ffn.kind).tensor_needs(spec.ffn)
        return needs

    def forward(self, h: torch.Tensor, pending, step, memory: int, writes: bool):
        n = h.shape[0]
        if h.shape[1] != self.streams * self.hidden:
            raise ValueError(f"a block of {self.streams} streams was handed a residual of {h.shape[1]} elements a token")
        x = self.env.workspace.get("normed", n, self.hidden, self.env.dtype)
        write_and_read(h, self.streams, self.hidden, pending, self.mixer_streams.read, self.pre_mixer, x)
        pending = (self.mixer.forward(x, step, memory, writes), self.mixer_streams)
        if self.ffn is None:
            return pending
        write_and_read(h, self.streams, self.hidden, pending, self.ffn_streams.read, self.pre_ffn, x)
        return (self.ffn.forward(x, step), self.ffn_streams)


register("block", "streams", StreamsBlock)
