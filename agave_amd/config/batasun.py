"""Typed configuration of the Batasun decoder, read from config.json's own keys.

config.json: ``architecture`` ("Batasun"), ``vocab``, ``width``, ``norm.eps`` and ``layers``, a list whose entries
give ``type`` (the mixer: ``latent_attention`` or ``mamba2``), ``mixer`` (its sizes and constants) and ``mlp``
(``{"kind": "moe", ...}`` or null).  Tensor names: ``embed``, ``embed.norm``, ``l<i>.norm1|norm2``, ``l<i>.mix.*``,
``l<i>.mlp.*``, ``final.norm``, ``head``.

The embedding rows pass the model's norm first.  A layer has no norm in front of a sublayer and one behind it:
``x += rms(mixer(x)) (1 + w1);  x += rms(ff(x)) (1 + w2)``.

``latent_attention``  queries through a latent of ``q_rank`` with its own norm; keys and values from one cached
                      latent row of ``kv_rank`` (normed) plus ``rot_dim`` rotated elements shared by the heads; per
                      head ``dim`` plain and ``rot_dim`` rotated query/key elements and values of ``vdim``; causal
                      softmax of ``scale * q.k``; the heads times ``sigmoid(W_g x)``.  With ``kv_from: j`` the layer
                      has no latent projection of its own and reads layer j's cached rows.
``mamba2``            a state-space mixer: ``heads`` of ``vdim``, a state of ``state`` rows per head, ``groups`` of
                      B and C, a causal convolution of ``conv`` taps with a bias, one decay per head and token, a
                      gate before a norm in ``norm_groups`` parts.

Feed-forward ``moe``: ``router.experts`` experts of size ``expert.ff`` whose gate is capped at ``expert.limit`` and
whose up value is clamped to it, ``g sigmoid(1.702 g) (u + 1)``; the ``router.top`` largest logits (with a bias)
choose, weighted by the softmax over the chosen; a shared expert (``shared.ff``, ``shared.limit``) times a sigmoid
gate per token.

The design has no bound on positions; :data:`POSITIONS` is what the engine is told.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Iterable, List, Optional, Tuple

from .errors import ConfigError
from .rilenex import _int, _num, _obj
from .spec import (GatedFfnSpec, LatentAttentionSpec, LayerSpec, Mamba2Spec, ModelSpec, NormSpec, PositionSpec,
                   RoutedFfnSpec, RunEntry)

POSITIONS = 1 << 20           # the longest sequence the engine is told of (no tensor or constant depends on it)
SWISH_ALPHA = 1.702           # g sigmoid(SWISH_ALPHA g): the design fixes it


@dataclass(frozen=True)
class BatasunLatent:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot_base: float
    rot_dims: int
    kv_from: Optional[int] = None


@dataclass(frozen=True)
class BatasunMamba:
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int


@dataclass(frozen=True)
class BatasunMoe:
    experts: int
    top: int
    ff: int
    limit: float
    shared_ff: Optional[int]
    shared_limit: float


@dataclass(frozen=True)
class BatasunLayer:
    type: str                          # "latent_attention" | "mamba2"
    mixer: object                      # BatasunLatent | BatasunMamba
    mlp: Optional[BatasunMoe]


@dataclass(frozen=True)
class BatasunConfig:
    vocab: int
    width: int
    eps: float
    layers: Tuple[BatasunLayer, ...]

    architecture = "Batasun"

    # ------------------------------------------------------------------ parse
    @classmethod
    def from_dict(cls, raw: dict) -> "BatasunConfig":
        vocab, width = _int(raw, "vocab", "top level"), _int(raw, "width", "top level")
        eps = _num(_obj(raw, "norm", "top level"), "eps", "norm", positive=True)
        entries = raw.get("layers")
        if not isinstance(entries, list) or not entries:
            raise ConfigError("config.json: 'layers' must be a list with at least one layer")
        layers: List[BatasunLayer] = []
        for i, e in enumerate(entries):
            where = f"layers[{i}]"
            if not isinstance(e, dict):
                raise ConfigError(f"config.json: {where} must be an object")
            kind = e.get("type")
            m = _obj(e, "mixer", where)
            mw = where + ".mixer"
            if kind == "latent_attention":
                rot = _obj(m, "rot", mw)
                rot_dim = _int(m, "rot_dim", mw)
                dims = _int(rot, "dims", mw + ".rot", least=2)
                if dims % 2 or dims > rot_dim:
                    raise ConfigError(f"config.json: {mw}.rot: 'dims' ({dims}) must be even and at most rot_dim ({rot_dim})")
                kv_from = _int(m, "kv_from", mw, least=0) if m.get("kv_from") is not None else None
                mixer = BatasunLatent(_int(m, "heads", mw), _int(m, "dim", mw), rot_dim, _int(m, "vdim", mw),
                                      _int(m, "q_rank", mw), _int(m, "kv_rank", mw), _num(m, "scale", mw),
                                      _num(rot, "base", mw + ".rot", positive=True), dims, kv_from)
            elif kind == "mamba2":
                heads, groups = _int(m, "heads", mw), _int(m, "groups", mw)
                if heads % groups:
                    raise ConfigError(f"config.json: {mw}: heads ({heads}) is not a multiple of groups ({groups})")
                mixer = BatasunMamba(heads, _int(m, "vdim", mw), _int(m, "state", mw), groups, _int(m, "conv", mw),
                                     _int(m, "norm_groups", mw))
                if (mixer.heads * mixer.vdim) % mixer.norm_groups:
                    raise ConfigError(f"config.json: {mw}: heads * vdim ({mixer.heads * mixer.vdim}) does not split into "
                                      f"{mixer.norm_groups} equal parts (norm_groups)")
            else:
                raise ConfigError(f"config.json: {where}: unknown layer type {kind!r} (latent_attention, mamba2)")
            layers.append(BatasunLayer(kind, mixer, cls._mlp(e.get("mlp"), where + ".mlp")))
        for i, layer in enumerate(layers):
            j = layer.mixer.kv_from if layer.type == "latent_attention" else None
            if j is None:
                continue
            mw = f"layers[{i}].mixer"
            if j >= i:
                raise ConfigError(f"config.json: {mw}: kv_from ({j}) must name an earlier layer")
            src = layers[j]
            if src.type != "latent_attention" or src.mixer.kv_from is not None:
                raise ConfigError(f"config.json: {mw}: kv_from ({j}) names a layer without a latent projection of its own")
            a, b = layer.mixer, src.mixer
            if (a.kv_rank, a.rot_dim, a.rot_base, a.rot_dims) != (b.kv_rank, b.rot_dim, b.rot_base, b.rot_dims):
                raise ConfigError(f"config.json: {mw}: kv_rank, rot_dim and rot must equal those of layer {j}, whose "
                                  f"latent rows it reads")
        return cls(vocab, width, eps, tuple(layers))

    @staticmethod
    def _mlp(mlp, where: str) -> Optional[BatasunMoe]:
        if mlp is None:
            return None
        if not isinstance(mlp, dict):
            raise ConfigError(f"config.json: {where} must be null or an object")
        if mlp.get("kind") != "moe":
            raise ConfigError(f"config.json: {where}: unknown kind {mlp.get('kind')!r} (moe)")
        r = _obj(mlp, "router", where)
        experts, top = _int(r, "experts", where + ".router"), _int(r, "top", where + ".router")
        if top > experts:
            raise ConfigError(f"config.json: {where}.router: top ({top}) exceeds the {experts} experts")
        ex = _obj(mlp, "expert", where)
        ff, limit = _int(ex, "ff", where + ".expert"), _num(ex, "limit", where + ".expert", positive=True)
        shared_ff, shared_limit = None, limit
        if mlp.get("shared") is not None:
            sh = _obj(mlp, "shared", where)
            shared_ff = _int(sh, "ff", where + ".shared")
            shared_limit = _num(sh, "limit", where + ".shared", positive=True)
        return BatasunMoe(experts, top, ff, limit, shared_ff, shared_limit)

    # ------------------------------------------------------------------ export
    def to_dict(self) -> dict:
        """config.json content that parses back to this configuration."""
        out = []
        for layer in self.layers:
            m = layer.mixer
            if layer.type == "latent_attention":
                mixer = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "q_rank": m.q_rank,
                         "kv_rank": m.kv_rank, "scale": m.scale, "rot": {"base": m.rot_base, "dims": m.rot_dims}}
                if m.kv_from is not None:
                    mixer["kv_from"] = m.kv_from
            else:
                mixer = {"heads": m.heads, "vdim": m.vdim, "state": m.state, "groups": m.groups, "conv": m.conv,
                         "norm_groups": m.norm_groups}
            f = layer.mlp
            mlp = None
            if f is not None:
                mlp = {"kind": "moe", "expert": {"ff": f.ff, "limit": f.limit}, "router": {"experts": f.experts, "top": f.top}}
                if f.shared_ff is not None:
                    mlp["shared"] = {"ff": f.shared_ff, "limit": f.shared_limit}
            out.append({"type": layer.type, "mixer": mixer, "mlp": mlp})
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
                "layers": out}

    # ------------------------------------------------------------------ spec
    def model_spec(self, tensor_names: Optional[Iterable[str]] = None) -> ModelSpec:
        e, eps = self.width, self.eps

        def norm(name: str) -> NormSpec:
            return NormSpec("rmsnorm", e, eps, name, add_one=True)

        layers: List[LayerSpec] = []
        order: List[RunEntry] = []
        for i, layer in enumerate(self.layers):
            p, m = f"l{i}.mix.", layer.mixer
            memory, writes = i, True
            if layer.type == "latent_attention":
                own = m.kv_from is None
                mixer = LatentAttentionSpec(
                    kind="latent_attention", hidden=e, n_heads=m.heads, head_dim=m.dim, rot_dim=m.rot_dim, v_head_dim=m.vdim,
                    q_rank=m.q_rank, kv_rank=m.kv_rank, scale=m.scale, norm_eps=eps,
                    position=PositionSpec("rope", rotary_dim=m.rot_dims, theta=m.rot_base),
                    q_down=p + "dq", q_norm=p + "dq.norm", q_up=p + "uq", kv_down=p + "dkv" if own else "",
                    kv_norm=p + "dkv.norm" if own else "", k_up=p + "uk", v_up=p + "uv", gate_proj=p + "g", o_proj=p + "o")
                if not own:       # the layer reads the memory of the layer it names, and appends nothing
                    memory, writes = m.kv_from, False
            else:
                mixer = Mamba2Spec(
                    kind="mamba2", hidden=e, n_heads=m.heads, v_head_dim=m.vdim, state=m.state, groups=m.groups,
                    conv_taps=m.conv, norm_groups=m.norm_groups, norm_eps=eps, in_proj=p + "in", conv=p + "conv",
                    conv_bias=p + "conv.b", dt_bias=p + "dt_bias", a_log=p + "A_log", d_skip=p + "D", out_norm=p + "norm",
                    o_proj=p + "o")
            f, fp = layer.mlp, f"l{i}.mlp."
            ffn = None
            if f is not None:
                shared = None
                if f.shared_ff is not None:
                    shared = GatedFfnSpec(kind="gated_dense", hidden=e, intermediate=f.shared_ff, activation="swish_clamped",
                                          gate_proj=fp + "shared.gate", up_proj=fp + "shared.up", down_proj=fp + "shared.down",
                                          act_limit=f.shared_limit, act_alpha=SWISH_ALPHA)
                ffn = RoutedFfnSpec(kind="routed", hidden=e, intermediate=f.ff, n_experts=f.experts, n_identity=0, top=f.top,
                                    activation="swish_clamped", router=fp + "router", correction=fp + "router.b",
                                    expert_prefix=fp + "e", shared=shared, score="softmax_top",
                                    shared_gate=fp + "shared.sg" if shared is not None else "", act_limit=f.limit,
                                    act_alpha=SWISH_ALPHA)
            layers.append(LayerSpec(kind="postnorm", mixer=mixer, ffn=ffn, post_mixer_norm=norm(f"l{i}.norm1"),
                                    post_ffn_norm=norm(f"l{i}.norm2") if ffn is not None else None))
            order.append(RunEntry(i, memory, writes))
        return ModelSpec(
            architecture=self.architecture, vocab_size=self.vocab, hidden=e, embed_weight="embed", embed_scale=1.0,
            layers=layers, order=order, final_norm=norm("final.norm"), head_weight="head", max_context=POSITIONS,
            bos_token_id=None, eos_token_ids=(), embed_norm=norm("embed.norm"),
            # a tensor that no part asks for (the second norm of a layer without a feed-forward, say) is passed over
            tensor_scope=())
