"""Architecture-neutral description of a decoder: what the engine builds from.

An architecture's typed configuration (for instance :class:`Gemma3Config`) turns
itself into a :class:`ModelSpec`: a list of layers, each naming its mixer, its
feed-forward, its norms and its position encoding *by kind* with their sizes and
constants as plain data, plus the order in which the layers run.  The engine
looks every ``kind`` up in the part registries (``agave_amd.parts``); no part
knows which model it is in, and no size lives anywhere but here.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple


@dataclass(frozen=True)
class NormSpec:
    """A normalisation over the last axis.  ``weight`` is the tensor's full name."""
    kind: str                      # "rmsnorm" | "layernorm"
    size: int
    eps: float
    weight: str
    add_one: bool = False          # gain = 1 + w instead of w
    bias: str = ""                 # layernorm: the tensor added after the weight; "": none
    scale_by: str = ""             # a vector that multiplies the norm's result element by element (a layer scale); "": none
    mult: float = 1.0              # a number that multiplies the norm's result (a multiplier on a residual branch)


@dataclass(frozen=True)
class PositionSpec:
    """A position encoding applied to queries and keys inside a mixer."""
    kind: str                      # "rope" | "rope_yarn" | "none"
    rotary_dim: int = 0
    theta: float = 0.0
    factor: float = 1.0            # linear scaling: positions are divided by it
    interleaved: bool = False      # the rotated pairs are (2i, 2i+1) instead of (i, i + rotary_dim/2)
    # "rope_yarn": pair i's frequency f_i = theta^(-2i/rotary_dim) becomes f_i / yarn_factor * r_i + f_i (1 - r_i) with
    # r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), lo = max(floor(d(yarn_fast)), 0), hi = min(ceil(d(yarn_slow)),
    # rotary_dim - 1), d(t) = rotary_dim ln(yarn_original / (2 pi t)) / (2 ln theta); sine and cosine are multiplied by
    # yarn_magnitude_slope ln(yarn_factor) + 1
    yarn_factor: float = 1.0
    yarn_original: int = 0
    yarn_fast: float = 32.0
    yarn_slow: float = 1.0
    yarn_magnitude_slope: float = 0.1


@dataclass(frozen=True)
class MixerSpec:
    """Base of the token mixers.  ``kind`` selects the implementation."""
    kind: str


@dataclass(frozen=True)
class AttentionSpec(MixerSpec):
    hidden: int = 0
    n_heads: int = 0
    n_kv_heads: int = 0
    head_dim: int = 0
    scale: float = 1.0             # multiplies q.k
    window: Optional[int] = None   # None: all earlier keys; W: keys p-W+1 .. p
    position: PositionSpec = PositionSpec("none")
    q_norm: Optional[NormSpec] = None
    k_norm: Optional[NormSpec] = None
    q_proj: str = ""
    k_proj: str = ""
    v_proj: str = ""
    o_proj: str = ""
    q_bias: str = ""               # names of the projections' bias vectors; "": none
    k_bias: str = ""
    v_bias: str = ""
    o_bias: str = ""


@dataclass(frozen=True)
class TalkingAttentionSpec(MixerSpec):
    """Softmax attention whose heads' scores are mixed by a matrix before the softmax, with keys
    and values of different sizes, an optional short convolution behind the projections, an
    optional gate per head on the output, and keys limited to the query's own chunk of positions."""
    hidden: int = 0
    n_heads: int = 0
    n_kv_heads: int = 0
    head_dim: int = 0              # queries and keys
    v_head_dim: int = 0            # values
    scale: float = 1.0             # multiplies q.k
    chunk: Optional[int] = None    # None: all earlier keys; C: keys j <= i with j // C == i // C
    conv_taps: int = 0             # 0: no convolution
    position: PositionSpec = PositionSpec("none")
    q_norm: Optional[NormSpec] = None
    k_norm: Optional[NormSpec] = None
    q_proj: str = ""
    k_proj: str = ""
    v_proj: str = ""
    o_proj: str = ""
    q_conv: str = ""               # [channels, taps], the last column is the current token's
    k_conv: str = ""
    v_conv: str = ""
    talk: str = ""                 # [heads, heads]: score_h <- sum_g talk[h, g] score_g; "": none
    gate_proj: str = ""            # [heads, hidden]: head h's output times sigmoid(gate_proj x)_h; "": none


@dataclass(frozen=True)
class ScoreBiasSpec:
    """What is added to an attention score as a function of the distance n = i - j between query and key.

    ``"none"``;  ``"slopes"``: -slope_h n with slope_h = 2^(-slope_log2 (h + 1) / heads);
    ``"buckets"``: table[bucket(n), h] for a learned table of B rows, with
    bucket(n) = n for n < B // 2, else min(B - 1, B // 2 + floor(ln(n / (B // 2)) / ln(max_distance / (B // 2)) (B - B // 2)))."""
    kind: str = "none"
    slope_log2: float = 8.0
    table: str = ""                # [buckets, heads]
    buckets: int = 0
    max_distance: int = 0


@dataclass(frozen=True)
class BiasedAttentionSpec(MixerSpec):
    """Softmax attention without a rotation whose scores get a bias by distance, with keys and values of
    different sizes, a window, first positions that stay visible, an optional sink in the softmax's
    denominator and an optional sigmoid gate on the concatenated heads.  Without ``k_proj`` and ``v_proj``
    the mixer has no keys and values of its own and reads the memory its run-order entry names.

    Optional besides: biases on the q, k and v products; an RMS norm over the whole row of q and of k (all heads side by
    side, one weight per element; ``q_row_norm``, ``k_row_norm``), before a rotation of the heads' first elements
    (``position``); a cap on the scaled scores, ``softcap * tanh(score / softcap)``, before the bias; and chunks
    instead of (or besides) a window: a query sees only keys of its own chunk of ``chunk`` positions, counted from the
    sequence's first."""
    hidden: int = 0
    n_heads: int = 0
    n_kv_heads: int = 0
    head_dim: int = 0              # queries and keys
    v_head_dim: int = 0            # values
    scale: float = 1.0             # multiplies q.k (not the bias)
    window: Optional[int] = None   # None: all earlier keys; W: keys i-W+1 .. i
    keep_first: int = 0            # keys j < keep_first stay visible whatever the window
    bias: ScoreBiasSpec = ScoreBiasSpec()
    sink: str = ""                 # [heads]: exp(sink_h) joins the denominator; "": none
    gate_proj: str = ""            # [heads * v_head_dim, hidden]: heads times sigmoid(gate_proj x); "": none
    q_proj: str = ""
    k_proj: str = ""
    v_proj: str = ""
    o_proj: str = ""
    q_bias: str = ""               # names of the products' bias vectors; "": none
    k_bias: str = ""
    v_bias: str = ""
    q_row_norm: Optional[NormSpec] = None      # RMS norm over the whole q row [heads * head_dim]
    k_row_norm: Optional[NormSpec] = None      # over the whole k row [kv heads * head_dim]
    position: PositionSpec = PositionSpec("none")
    softcap: float = 0.0           # > 0: score <- softcap * tanh(score / softcap)
    chunk: Optional[int] = None    # None: no chunks; C: only keys j with j // C == i // C


@dataclass(frozen=True)
class LatentAttentionSpec(MixerSpec):
    """Causal softmax attention whose keys and values are made from one small latent row per position.

    ``cq = rms(q_down x) * q_norm``, ``q = q_up cq`` (per head ``head_dim`` plain elements, then ``rot_dim`` that
    are rotated); ``kv_down x = [c' | r]`` with ``c = rms(c') * kv_norm`` (``kv_rank`` elements) and ``r``
    (``rot_dim`` elements, rotated, shared by the heads).  Head h's key is ``[k_up_h c | r]``, its value
    ``v_up_h c``; the score is ``scale * q . k``.  The cache holds ``[c | r]`` per position and nothing per head.
    The heads side by side are multiplied by ``sigmoid(gate_proj x)`` where a gate is named.  Without ``kv_down``
    the mixer reads the latent rows of the memory its run-order entry names, with its own ``k_up`` and ``v_up``.
    ``position`` rotates the first ``rotary_dim`` of the ``rot_dim`` elements (pairs i, i + rotary_dim / 2)."""
    hidden: int = 0
    n_heads: int = 0
    head_dim: int = 0              # elements of a query/key head that are not rotated
    rot_dim: int = 0               # elements that are (queries: per head; keys: one part for all heads)
    v_head_dim: int = 0
    q_rank: int = 0
    kv_rank: int = 0
    scale: float = 1.0
    norm_eps: float = 1e-5         # of the latents' norms
    position: PositionSpec = PositionSpec("none")
    q_down: str = ""               # [q_rank, hidden]
    q_norm: str = ""               # [q_rank]
    q_up: str = ""                 # [heads * (head_dim + rot_dim), q_rank]
    kv_down: str = ""              # [kv_rank + rot_dim, hidden]; "": another memory's latent rows are read
    kv_norm: str = ""              # [kv_rank]
    k_up: str = ""                 # [heads * head_dim, kv_rank]
    v_up: str = ""                 # [heads * v_head_dim, kv_rank]
    gate_proj: str = ""            # [heads * v_head_dim, hidden]; "": no gate
    o_proj: str = ""               # [hidden, heads * v_head_dim]


@dataclass(frozen=True)
class Mamba2Spec(MixerSpec):
    """A state-space mixer with one decay per head and token (state [heads, state, v_head_dim]).

    ``in_proj x = [z | xs | B | C | dt]`` (``heads * v_head_dim`` twice, ``groups * state`` twice, ``heads``);
    ``xs, B, C`` pass one short causal convolution with a bias and SiLU; ``dt = softplus(dt + dt_bias)``;
    head h (group ``h // (heads / groups)``): ``S <- exp(-exp(a_log_h) dt) S + dt B xs^T``, ``y = S^T C + d_skip_h xs``;
    ``y * silu(z)`` is divided by its root mean square in ``norm_groups`` equal parts, times ``out_norm``."""
    hidden: int = 0
    n_heads: int = 0
    v_head_dim: int = 0
    state: int = 0
    groups: int = 1
    conv_taps: int = 1
    norm_groups: int = 1
    norm_eps: float = 1e-5
    in_proj: str = ""
    conv: str = ""                 # [heads * v_head_dim + 2 * groups * state, taps], the last column is the current token's
    conv_bias: str = ""            # "": none
    dt_bias: str = ""              # [heads]
    a_log: str = ""                # [heads]
    d_skip: str = ""               # [heads]
    out_norm: str = ""             # [heads * v_head_dim]
    o_proj: str = ""


@dataclass(frozen=True)
class GatedDeltaSpec(MixerSpec):
    """Delta rule with a decay per head and key channel (state [heads, head_dim, v_head_dim])."""
    hidden: int = 0
    n_heads: int = 0               # value heads, and states
    n_kv_heads: int = 0            # query/key heads; head h reads head h // (n_heads / n_kv_heads)
    head_dim: int = 0
    v_head_dim: int = 0
    conv_taps: int = 0
    decay_rank: int = 0            # inner size of the decay's two projections
    gate_rank: int = 0             # inner size of the output gate's two projections
    norm_eps: float = 1e-5         # of the read-out's norm
    unit_eps: float = 1e-6         # q and k become x / sqrt(sum(x^2) + unit_eps) per head
    q_proj: str = ""
    k_proj: str = ""
    v_proj: str = ""
    o_proj: str = ""
    q_conv: str = ""
    k_conv: str = ""
    v_conv: str = ""
    beta_proj: str = ""            # [heads, hidden]
    decay_in: str = ""             # [decay_rank, hidden]
    decay_out: str = ""            # [heads * head_dim, decay_rank]
    decay_bias: str = ""           # [heads * head_dim]
    decay_log: str = ""            # [heads]: the rate is exp of it
    gate_in: str = ""              # [gate_rank, hidden]
    gate_out: str = ""             # [heads * v_head_dim, gate_rank]
    out_norm: str = ""             # [v_head_dim], shared by the heads


@dataclass(frozen=True)
class Hgrn2Spec(MixerSpec):
    """Linear attention whose forget gate also sets what is written (state [heads, head_dim, v_head_dim])."""
    hidden: int = 0
    n_heads: int = 0
    head_dim: int = 0
    v_head_dim: int = 0
    norm_eps: float = 1e-5
    q_proj: str = ""
    f_proj: str = ""
    f_bias: str = ""
    lower: str = ""                # [heads * head_dim]: the forget gate's lower bound
    v_proj: str = ""
    o_proj: str = ""
    out_norm: str = ""             # [v_head_dim], shared by the heads


@dataclass(frozen=True)
class RglruSpec(MixerSpec):
    """A gated linear recurrence per channel (state [width]) beside a GELU branch.

    ``y = gelu_tanh(y_proj x + y_bias)``; ``u = conv(x_proj x + x_bias)`` (a short causal convolution per channel with a
    bias, no activation); in each of ``blocks`` equal parts b of the channels ``r = sigmoid(r_gate[b] u_b + r_bias[b])``
    and ``g = sigmoid(i_gate[b] u_b + i_bias[b])``; ``a = exp(-decay_scale r softplus(lam))``;
    ``S <- a S + sqrt(1 - a^2) g u`` from S = 0; the result is ``o_proj (S y)``."""
    hidden: int = 0
    width: int = 0
    blocks: int = 1
    conv_taps: int = 1
    decay_scale: float = 8.0
    y_proj: str = ""
    y_bias: str = ""
    x_proj: str = ""
    x_bias: str = ""
    conv: str = ""                 # [width, taps], the last column is the current token's
    conv_bias: str = ""
    r_gate: str = ""               # [blocks, width / blocks, width / blocks], [out, in] inside a block
    r_bias: str = ""               # [blocks, width / blocks]
    i_gate: str = ""
    i_bias: str = ""
    lam: str = ""                  # [width]
    o_proj: str = ""


@dataclass(frozen=True)
class ParallelMixerSpec(MixerSpec):
    """Mixers side by side on the same input; the result is the sum of ``scales[i] * branches[i]``."""
    branches: Tuple[MixerSpec, ...] = ()
    scales: Tuple[float, ...] = ()


@dataclass(frozen=True)
class FeedForwardSpec:
    kind: str


@dataclass(frozen=True)
class DenseFfnSpec(FeedForwardSpec):
    """``W_down act(W_up x)``.  ``act_params`` names a small tensor of the activation's learned
    numbers where it has some (xielu: two)."""
    hidden: int = 0
    intermediate: int = 0
    activation: str = "gelu_tanh"
    up_proj: str = ""
    down_proj: str = ""
    act_params: str = ""


@dataclass(frozen=True)
class GatedFfnSpec(FeedForwardSpec):
    hidden: int = 0
    intermediate: int = 0
    activation: str = "gelu_tanh"
    gate_proj: str = ""
    up_proj: str = ""
    down_proj: str = ""
    gate_bias: str = ""            # names of the products' bias vectors; "": none
    up_bias: str = ""
    down_bias: str = ""
    # ``swish_clamped``: g = min(gate, act_limit), u = clamp(up, -act_limit, act_limit), g sigmoid(act_alpha g) (u + 1)
    act_limit: float = 0.0
    act_alpha: float = 1.0


@dataclass(frozen=True)
class RoutedFfnSpec(FeedForwardSpec):
    """A mixture of gated experts ``W_down (act(W_gate x) * (W_up x))``.  The router has ``n_experts +
    n_identity`` outputs; the last ``n_identity`` stand for experts whose result is their input.  Scores are
    the softmax over all outputs; the ``top`` outputs with the largest score + correction are chosen, among
    the ``keep_groups`` best of ``groups`` equal groups of neighbouring outputs (a group counts by its largest
    score + correction); a chosen expert's weight is its score times ``route_scale``.  ``shared``: an expert
    that every token runs through, added; with ``shared_gate`` [1, hidden] it is first multiplied by
    ``sigmoid(shared_gate . x)``, one number per token.

    ``score="softmax_top"`` instead: the router's logits plus ``correction`` (a bias of the logits here) decide, the
    ``top`` largest are chosen, and the weights are the softmax over the chosen logits alone, times ``route_scale``
    (no groups).  ``score="sigmoid"``: the scores are ``sigmoid`` of the logits, each on its own; choice and groups as
    with ``softmax_all``.  ``group_top``: a group counts by the sum of its this many largest scores + correction (1: by
    its largest).  ``normalise``: the chosen experts' weights are divided by their sum + 1e-20 (before ``route_scale``).
    ``act_limit`` and ``act_alpha`` are the activation's numbers where it has some
    (``swish_clamped``, see :class:`GatedFfnSpec`)."""
    hidden: int = 0
    intermediate: int = 0          # of every expert
    n_experts: int = 0
    n_identity: int = 0
    top: int = 1
    groups: int = 1
    keep_groups: int = 1
    route_scale: float = 1.0
    activation: str = "silu"
    router: str = ""               # [n_experts + n_identity, hidden]
    correction: str = ""           # [n_experts + n_identity]; "": none
    expert_prefix: str = ""        # expert i's matrices are expert_prefix + f"{i}." + gate | up | down
    gate_name: str = "gate"
    up_name: str = "up"
    down_name: str = "down"
    shared: Optional[GatedFfnSpec] = None
    score: str = "softmax_all"     # | "softmax_top" | "sigmoid"
    group_top: int = 1
    normalise: bool = False
    shared_gate: str = ""          # [1, hidden]; "": the shared expert is added as it is
    act_limit: float = 0.0
    act_alpha: float = 1.0


@dataclass(frozen=True)
class LayerSpec:
    """One block.  ``kind`` selects the arrangement of the parts:

    ``"sandwich"``: h += post_mixer_norm(mixer(pre_mixer_norm(h)));
                    h += post_ffn_norm(ffn(pre_ffn_norm(h)))
    ``"prenorm"``:  the same without the two post norms.
    ``"postnorm"``: h += post_mixer_norm(mixer(h));  h += post_ffn_norm(ffn(h)): the sublayers read the stream itself.
    ``"streams"``:  the residual is ``ModelSpec.streams`` rows x_1 .. x_S per token; a sublayer reads
                    u = sum_s read[s] x_s, computes y = sublayer(pre_norm(u)), and writes, all streams at once,
                    x_t <- sum_s mix[s, t] x_s + write[t] y (``mixer_streams``, ``ffn_streams``).
    """
    kind: str
    mixer: MixerSpec
    ffn: Optional[FeedForwardSpec]
    pre_mixer_norm: Optional[NormSpec] = None
    post_mixer_norm: Optional[NormSpec] = None
    pre_ffn_norm: Optional[NormSpec] = None
    post_ffn_norm: Optional[NormSpec] = None
    mixer_streams: Optional["StreamMixSpec"] = None
    ffn_streams: Optional["StreamMixSpec"] = None


@dataclass(frozen=True)
class StreamMixSpec:
    """How one sublayer reads and writes several residual streams (tensor names)."""
    streams: int
    read: str                      # [streams]: the sublayer's input is sum_s read[s] x_s
    write: str                     # [streams]: stream t receives write[t] times the sublayer's result
    mix: str                       # [streams, streams], indexed [from, to]: the streams are mixed as the result is added


@dataclass(frozen=True)
class RunEntry:
    """One entry of the run order.  ``layer`` indexes ``ModelSpec.layers``;
    ``memory`` names the cache (and fixed-size state) this run of the layer uses;
    two entries with the same ``memory`` share it, and only entries with
    ``writes`` append to it."""
    layer: int
    memory: int
    writes: bool = True


@dataclass
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden: int
    embed_weight: str
    embed_scale: float
    layers: List[LayerSpec]
    order: List[RunEntry]
    final_norm: Optional[NormSpec]
    head_weight: Optional[str]           # None: tied to the embedding
    max_context: int
    bos_token_id: Optional[int] = None
    eos_token_ids: Tuple[int, ...] = ()
    # Name prefixes of the tensors that are this model's own.  A checkpoint's tensor that no
    # part asked for is an error under one of them and is passed over elsewhere (a vision
    # tower beside a text decoder).  None: every name in the checkpoint is the model's.
    tensor_scope: Optional[Tuple[str, ...]] = None
    # what is done to the logits after the output product: multiplied by ``logit_scale``, then
    # soft-capped to +-``logit_softcap`` (cap * tanh(x / cap)) if that is above zero
    logit_scale: float = 1.0
    logit_softcap: float = 0.0
    embed_norm: Optional[NormSpec] = None    # a norm on the embedding rows before the first layer
    # > 0: the residual is this many streams per token (layers of kind "streams"), all equal to the embedding row at
    # the start; their sum enters the final norm.  0: one stream, the ordinary residual sum.
    streams: int = 0
    extra: Dict[str, object] = field(default_factory=dict)

    def default_order(self) -> List[RunEntry]:
        return [RunEntry(i, i, True) for i in range(len(self.layers))]
