"""Typed configuration of the Duperax decoder, read from config.json's own keys.

config.json: ``architecture`` ("Duperax"), ``vocab``, ``width``, ``norm.eps``, ``logit_scale``, ``streams`` (the number of
residual streams; absent: one ordinary residual), ``loop`` (``start``, ``stop``, ``times``: layers start .. stop - 1 run
that many times in a row, each pass with its own cache and state) and ``layers``, a list whose entries give ``type``
(the mixer: ``attention``, ``attention_2`` or ``rglru``), ``mixer`` (its sizes and constants) and ``mlp``
(``{"kind": "dense", "ff": n, "limit": L}``, ``{"kind": "moe", ...}`` or null).
Tensor names: ``embed``, ``l<i>.norm1|norm2`` (each with ``.b``), ``l<i>.hc1|hc2.in|out|mix``, ``l<i>.mix.*``,
``l<i>.mlp.*``, ``final.norm`` (with ``.b``), ``head``.

A layer has a layer norm before each sublayer.  With one residual: ``x += mixer(norm1(x)); x += ff(norm2(x))``.  With S
streams ``x_1 .. x_S`` (all equal to the embedding row at first), sublayer q reads ``u = sum_s in_q[s] x_s`` and writes
``x_t <- sum_s mix_q[s, t] x_s + out_q[t] f(norm_q(u))`` for all t at once; the streams' sum enters the final norm.

Mixers: ``attention``: grouped softmax attention with keys of size ``dim`` and values of size ``vdim``, q and k divided by
the root mean square of their whole row (all heads) times a weight, no rotation, ``scale`` on q.k, a sliding window
``mask.size``.  ``attention_2``: the same with biases on q, k and v, a rotation of each head's first ``rot.dims``
elements (pairs (e, e + dims/2), base ``rot.base``, YaRN's frequencies and magnitude from ``rot.scaling``), a cap
``softcap * tanh(score / softcap)`` on the scaled scores, and chunks of ``mask.size`` positions instead of a window.
``rglru``: a gated linear recurrence per channel of ``width`` channels with block-diagonal gates (``blocks``) behind a
short convolution (``conv`` taps), beside a GELU branch.

Feed-forwards: ``dense``: ``g = min(W_g x, limit)``, ``u = clamp(W_u x, -limit, limit)``, ``W_d (g sigmoid(1.702 g) (u + 1))``;
``moe``: ``router.experts`` gated SiLU experts of size ``expert.ff``, ``router.top`` of them per token chosen by
sigmoid score + ``correction`` within the best ``groups.keep`` of ``groups.count`` groups (a group counts by the sum of
its two largest), weighted by their scores divided by the scores' sum.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Iterable, List, Optional, Tuple

from .errors import ConfigError
from .rilenex import _int, _num, _obj
from .spec import (BiasedAttentionSpec, GatedFfnSpec, LayerSpec, ModelSpec, NormSpec, PositionSpec, RglruSpec, RoutedFfnSpec,
                   RunEntry, ScoreBiasSpec, StreamMixSpec)

POSITIONS = 1 << 20           # the longest sequence the engine is told of (no tensor or constant depends on it)
SWISH_ALPHA = 1.702           # the dense feed-forward's g sigmoid(alpha g): the design fixes it
DECAY_SCALE = 8.0             # the recurrence's log a = -DECAY_SCALE r softplus(lam)
YARN_MAGNITUDE_SLOPE = 0.1    # sine and cosine times YARN_MAGNITUDE_SLOPE ln(factor) + 1
GROUP_TOP = 2                 # a group of experts counts by the sum of its two largest choice scores


@dataclass(frozen=True)
class DuperaxRotation:
    dims: int
    base: float
    factor: Optional[float] = None     # None: the plain frequencies
    original: int = 0
    fast: float = 32.0
    slow: float = 1.0


@dataclass(frozen=True)
class DuperaxAttention:
    type: str                          # "attention" | "attention_2"
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    size: Optional[int]                # the window (attention) or the chunk (attention_2); None: every earlier key
    rot: Optional[DuperaxRotation] = None
    softcap: float = 0.0


@dataclass(frozen=True)
class DuperaxRglru:
    width: int
    blocks: int
    conv: int
    type: str = "rglru"


@dataclass(frozen=True)
class DuperaxDense:
    ff: int
    limit: float


@dataclass(frozen=True)
class DuperaxMoe:
    experts: int
    top: int
    groups: int
    keep_groups: int
    ff: int


@dataclass(frozen=True)
class DuperaxLayer:
    mixer: object                      # DuperaxAttention | DuperaxRglru
    mlp: object                        # None | DuperaxDense | DuperaxMoe


@dataclass(frozen=True)
class DuperaxConfig:
    vocab: int
    width: int
    eps: float
    logit_scale: float
    streams: Optional[int]             # None: one ordinary residual
    loop: Optional[Tuple[int, int, int]]       # (start, stop, times)
    layers: Tuple[DuperaxLayer, ...]

    architecture = "Duperax"

    # ------------------------------------------------------------------ parse
    @classmethod
    def from_dict(cls, raw: dict) -> "DuperaxConfig":
        vocab, width = _int(raw, "vocab", "top level"), _int(raw, "width", "top level")
        eps = _num(_obj(raw, "norm", "top level"), "eps", "norm", positive=True)
        logit_scale = _num(raw, "logit_scale", "top level") if raw.get("logit_scale") is not None else 1.0
        streams = _int(raw, "streams", "top level") if raw.get("streams") is not None else None
        entries = raw.get("layers")
        if not isinstance(entries, list) or not entries:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        layers: List[DuperaxLayer] = []
        for i, e in enumerate(entries):
            where = f"layers[{i}]"
            if not isinstance(e, dict):
                raise ConfigError(f"config.json: {where} must be an object")
            kind = e.get("type")
            m = _obj(e, "mixer", where)
            mw = where + ".mixer"
            if kind in ("attention", "attention_2"):
                mixer = cls._attention(kind, m, mw)
            elif kind == "rglru":
                w, blocks = _int(m, "width", mw), _int(m, "blocks", mw) if m.get("blocks") is not None else 1
                if w % blocks:
                    raise ConfigError(f"config.json: {mw}: width ({w}) is not a multiple of blocks ({blocks})")
                mixer = DuperaxRglru(w, blocks, _int(m, "conv", mw))
            else:
                raise ConfigError(f"config.json: {where}: unknown layer type {kind!r} (attention, attention_2, rglru)")
            layers.append(DuperaxLayer(mixer, cls._mlp(e.get("mlp"), where + ".mlp")))
        loop = None
        if raw.get("loop") is not None:
            lp = _obj(raw, "loop", "top level")
            start, stop, times = _int(lp, "start", "loop", least=0), _int(lp, "stop", "loop", least=0), _int(lp, "times", "loop")
            if not start <= stop <= len(layers):
                raise ConfigError(f"config.json: loop: start ({start}) and stop ({stop}) must lie in order within the "
                                  f"{len(layers)} layers")
            loop = (start, stop, times)
        return cls(vocab, width, eps, logit_scale, streams, loop, tuple(layers))

    @staticmethod
    def _attention(kind: str, m: dict, mw: str) -> DuperaxAttention:
        heads, kv_heads = _int(m, "heads", mw), _int(m, "kv_heads", mw)
        if heads % kv_heads:
            raise ConfigError(f"config.json: {mw}: heads ({heads}) is not a multiple of kv_heads ({kv_heads})")
        dim = _int(m, "dim", mw)
        size = _int(_obj(m, "mask", mw), "size", mw + ".mask") if m.get("mask") is not None else None
        rot, softcap = None, 0.0
        if kind == "attention_2":
            if m.get("rot") is not None:
                r = _obj(m, "rot", mw)
                rw = mw + ".rot"
                dims = _int(r, "dims", rw, least=2)
                if dims % 2 or dims > dim:
                    raise ConfigError(f"config.json: {rw}: dims ({dims}) must be even and at most dim ({dim})")
                base = _num(r, "base", rw, positive=True)
                if r.get("scaling") is not None:
                    sc = _obj(r, "scaling", rw)
                    sw = rw + ".scaling"
                    rot = DuperaxRotation(dims, base, _num(sc, "factor", sw, positive=True), _int(sc, "original", sw),
                                          _num(sc, "fast", sw, positive=True), _num(sc, "slow", sw, positive=True))
                else:
                    rot = DuperaxRotation(dims, base)
            if m.get("softcap") is not None:
                softcap = _num(m, "softcap", mw, positive=True)
        return DuperaxAttention(kind, heads, kv_heads, dim, _int(m, "vdim", mw), _num(m, "scale", mw), size, rot, softcap)

    @staticmethod
    def _mlp(mlp, where: str):
        if mlp is None:
            return None
        if not isinstance(mlp, dict):
            raise ConfigError(f"config.json: {where} must be null or an object")
        kind = mlp.get("kind")
        if kind == "dense":
            return DuperaxDense(_int(mlp, "ff", where), _num(mlp, "limit", where, positive=True))
        if kind != "moe":
            raise ConfigError(f"config.json: {where}: unknown kind {kind!r} (dense, moe)")
        r = _obj(mlp, "router", where)
        rw = where + ".router"
        experts = _int(r, "experts", rw)
        groups, keep = 1, 1
        if r.get("groups") is not None:
            g = _obj(r, "groups", rw)
            groups, keep = _int(g, "count", rw + ".groups"), _int(g, "keep", rw + ".groups")
        if experts % groups or keep > groups:
            raise ConfigError(f"config.json: {rw}: {experts} experts must form {groups} equal groups, of which {keep} are kept")
        top = _int(r, "top", rw)
        if top > keep * (experts // groups):
            raise ConfigError(f"config.json: {rw}: top ({top}) exceeds the {keep * (experts // groups)} experts of the kept groups")
        return DuperaxMoe(experts, top, groups, keep, _int(_obj(mlp, "expert", where), "ff", where + ".expert"))

    # ------------------------------------------------------------------ export
    def to_dict(self) -> dict:
        """config.json content that parses back to this configuration."""
        out = []
        for layer in self.layers:
            m = layer.mixer
            if isinstance(m, DuperaxRglru):
                mixer = {"width": m.width, "blocks": m.blocks, "conv": m.conv}
            else:
                mixer = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale}
                if m.size is not None:
                    mixer["mask"] = {"size": m.size}
                if m.rot is not None:
                    mixer["rot"] = {"dims": m.rot.dims, "base": m.rot.base}
                    if m.rot.factor is not None:
                        mixer["rot"]["scaling"] = {"factor": m.rot.factor, "original": m.rot.original, "fast": m.rot.fast,
                                                   "slow": m.rot.slow}
                if m.softcap:
                    mixer["softcap"] = m.softcap
            f = layer.mlp
            if f is None:
                mlp = None
            elif isinstance(f, DuperaxDense):
                mlp = {"kind": "dense", "ff": f.ff, "limit": f.limit}
            else:
                mlp = {"kind": "moe", "expert": {"ff": f.ff},
                       "router": {"experts": f.experts, "top": f.top, "groups": {"count": f.groups, "keep": f.keep_groups}}}
            out.append({"type": m.type, "mixer": mixer, "mlp": mlp})
        d = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
             "logit_scale": self.logit_scale, "layers": out}
        if self.streams is not None:
            d["streams"] = self.streams
        if self.loop is not None:
            d["loop"] = {"start": self.loop[0], "stop": self.loop[1], "times": self.loop[2]}
        return d

    # ------------------------------------------------------------------ spec
    def run_order(self) -> List[int]:
        """The layers in the order they run: those before the loop, the loop's layers ``times`` times, the rest."""
        n = len(self.layers)
        if self.loop is None:
            return list(range(n))
        start, stop, times = self.loop
        return list(range(start)) + list(range(start, stop)) * times + list(range(stop, n))

    def model_spec(self, tensor_names: Optional[Iterable[str]] = None) -> ModelSpec:
        e, eps, S = self.width, self.eps, self.streams

        def norm(name: str) -> NormSpec:
            return NormSpec("layernorm", e, eps, name, bias=name + ".b")

        def streams(name: str) -> Optional[StreamMixSpec]:
            return StreamMixSpec(S, name + ".in", name + ".out", name + ".mix") if S is not None else None

        layers: List[LayerSpec] = []
        for i, layer in enumerate(self.layers):
            p = f"l{i}.mix."
            m = layer.mixer
            if isinstance(m, DuperaxRglru):
                mixer = RglruSpec(kind="rglru", hidden=e, width=m.width, blocks=m.blocks, conv_taps=m.conv,
                                  decay_scale=DECAY_SCALE, y_proj=p + "y", y_bias=p + "y.b", x_proj=p + "x", x_bias=p + "x.b",
                                  conv=p + "conv", conv_bias=p + "conv.b", r_gate=p + "ra", r_bias=p + "ra.b",
                                  i_gate=p + "ri", i_bias=p + "ri.b", lam=p + "lam", o_proj=p + "o")
            else:
                second = m.type == "attention_2"
                position = PositionSpec("none")
                if m.rot is not None and m.rot.factor is not None:
                    position = PositionSpec("rope_yarn", rotary_dim=m.rot.dims, theta=m.rot.base, yarn_factor=m.rot.factor,
                                            yarn_original=m.rot.original, yarn_fast=m.rot.fast, yarn_slow=m.rot.slow,
                                            yarn_magnitude_slope=YARN_MAGNITUDE_SLOPE)
                elif m.rot is not None:
                    position = PositionSpec("rope", rotary_dim=m.rot.dims, theta=m.rot.base)
                mixer = BiasedAttentionSpec(
                    kind="biased_attention", hidden=e, n_heads=m.heads, n_kv_heads=m.kv_heads, head_dim=m.dim,
                    v_head_dim=m.vdim, scale=m.scale, window=None if second else m.size, chunk=m.size if second else None,
                    bias=ScoreBiasSpec(kind="none"), q_proj=p + "q", k_proj=p + "k", v_proj=p + "v", o_proj=p + "o",
                    q_bias=p + "q.b" if second else "", k_bias=p + "k.b" if second else "", v_bias=p + "v.b" if second else "",
                    q_row_norm=NormSpec("rmsnorm", m.heads * m.dim, eps, p + "q.norm"),
                    k_row_norm=NormSpec("rmsnorm", m.kv_heads * m.dim, eps, p + "k.norm"),
                    position=position, softcap=m.softcap)
            f = layer.mlp
            fp = f"l{i}.mlp."
            if f is None:
                ffn = None
            elif isinstance(f, DuperaxDense):
                ffn = GatedFfnSpec(kind="gated_dense", hidden=e, intermediate=f.ff, activation="swish_clamped",
                                   gate_proj=fp + "gate", up_proj=fp + "up", down_proj=fp + "down", act_limit=f.limit,
                                   act_alpha=SWISH_ALPHA)
            else:
                ffn = RoutedFfnSpec(kind="routed", hidden=e, intermediate=f.ff, n_experts=f.experts, top=f.top, groups=f.groups,
                                    keep_groups=f.keep_groups, activation="silu", router=fp + "router",
                                    correction=fp + "correction", expert_prefix=fp + "e", score="sigmoid",
                                    group_top=GROUP_TOP, normalise=True)
            layers.append(LayerSpec(
                kind="streams" if S is not None else "prenorm", mixer=mixer, ffn=ffn, pre_mixer_norm=norm(f"l{i}.norm1"),
                pre_ffn_norm=norm(f"l{i}.norm2") if ffn is not None else None,
                mixer_streams=streams(f"l{i}.hc1"), ffn_streams=streams(f"l{i}.hc2") if ffn is not None else None))
        # every run of a layer has a memory of its own: a pass of the loop shares nothing with the pass before
        order = [RunEntry(layer, run, True) for run, layer in enumerate(self.run_order())]
        return ModelSpec(
            architecture=self.architecture, vocab_size=self.vocab, hidden=e, embed_weight="embed", embed_scale=1.0,
            layers=layers, order=order, final_norm=norm("final.norm"), head_weight="head", max_context=POSITIONS,
            bos_token_id=None, eos_token_ids=(), logit_scale=self.logit_scale, streams=S or 0,
            # a tensor that no part asks for (the second norm of a layer without a feed-forward, say) is passed over
            tensor_scope=())
