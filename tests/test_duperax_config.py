"""The Duperax configuration without a GPU: parser, round trip, errors that name the key, the spec and its run order,
the tensors the parts ask for, YaRN's frequencies, and the cache bookkeeping of chunks and of a layer that runs twice."""
import copy
import math

import pytest
import torch

import plain_duperax as P
from agave_amd.config import ConfigError, DuperaxConfig, find_architecture
from agave_amd.config.spec import BiasedAttentionSpec, GatedFfnSpec, RglruSpec, RoutedFfnSpec
from agave_amd.engine.model import tensor_needs


def sample():
    return P.config([
        P.attention2_layer(4, 2, 16, 8, 50, 8, base=500.0, factor=3.0, original=32, fast=16.0, slow=2.0, softcap=12.0,
                           mlp=P.moe(6, 2, 3, 2, 24)),
        P.rglru_layer(48, 3, 3, mlp=P.dense(56, limit=1.2)),
        P.attention_layer(3, 3, 8, 24, 37, mlp=None),
        P.rglru_layer(32, 1, 1, mlp=P.moe(4, 4, 1, 1, 16))],
        vocab=131, width=40, eps=2e-6, streams=3, loop=(1, 3, 2))


def test_found_by_its_name_and_round_trip():
    raw = sample()
    arch = find_architecture(raw)
    assert arch.name == "Duperax"
    cfg = arch.parse(raw)
    assert isinstance(cfg, DuperaxConfig) and cfg.to_dict() == raw
    assert DuperaxConfig.from_dict(cfg.to_dict()) == cfg
    assert cfg.streams == 3 and cfg.loop == (1, 3, 2) and cfg.logit_scale == 0.7
    assert cfg.layers[0].mixer.rot.factor == 3.0 and cfg.layers[0].mixer.softcap == 12.0 and cfg.layers[2].mixer.rot is None
    assert cfg.layers[1].mlp.limit == 1.2 and cfg.layers[2].mlp is None and cfg.layers[3].mixer.blocks == 1
    assert cfg.run_order() == P.run_order(raw) == [0, 1, 2, 1, 2, 3]


def test_what_is_not_there_does_not_exist():
    raw = sample()
    del raw["streams"], raw["loop"], raw["logit_scale"]
    del raw["layers"][0]["mixer"]["rot"]["scaling"], raw["layers"][0]["mixer"]["softcap"], raw["layers"][0]["mlp"]["router"]["groups"]
    cfg = DuperaxConfig.from_dict(raw)
    assert cfg.to_dict()["layers"][0]["mixer"]["rot"] == {"dims": 8, "base": 500.0}
    spec = cfg.model_spec()
    assert spec.streams == 0 and all(l.kind == "prenorm" and l.mixer_streams is None for l in spec.layers)
    assert [e.layer for e in spec.order] == [0, 1, 2, 3] and spec.logit_scale == 1.0
    m0 = spec.layers[0].mixer
    assert m0.position.kind == "rope" and m0.softcap == 0.0 and spec.layers[0].ffn.groups == 1
    needs = {n.name for n in tensor_needs(spec)}
    assert not any(".hc" in n for n in needs)
    del raw["layers"][0]["mixer"]["rot"]
    assert DuperaxConfig.from_dict(raw).model_spec().layers[0].mixer.position.kind == "none"


def test_spec_says_everything_the_parts_need():
    cfg = DuperaxConfig.from_dict(sample())
    spec = cfg.model_spec()
    # every run of a layer has a memory of its own
    assert [(e.layer, e.memory, e.writes) for e in spec.order] == [(0, 0, True), (1, 1, True), (2, 2, True), (1, 3, True), (2, 4, True), (3, 5, True)]
    assert spec.streams == 3 and spec.embed_norm is None and spec.embed_scale == 1.0 and spec.logit_scale == 0.7
    assert spec.final_norm.kind == "layernorm" and spec.final_norm.bias == "final.norm.b"
    assert all(l.kind == "streams" and l.pre_mixer_norm.kind == "layernorm" and l.post_mixer_norm is None for l in spec.layers)
    assert spec.layers[1].mixer_streams.mix == "l1.hc1.mix" and spec.layers[1].ffn_streams.read == "l1.hc2.in"
    assert spec.layers[2].ffn_streams is None and spec.layers[2].pre_ffn_norm is None
    m0, m1, m2 = spec.layers[0].mixer, spec.layers[1].mixer, spec.layers[2].mixer
    assert isinstance(m0, BiasedAttentionSpec) and (m0.chunk, m0.window, m0.softcap, m0.q_bias, m0.v_head_dim) == (50, None, 12.0, "l0.mix.q.b", 8)
    assert m0.position.kind == "rope_yarn" and (m0.position.rotary_dim, m0.position.theta, m0.position.yarn_factor) == (8, 500.0, 3.0)
    assert (m0.position.yarn_original, m0.position.yarn_fast, m0.position.yarn_slow, m0.position.yarn_magnitude_slope) == (32, 16.0, 2.0, 0.1)
    assert m0.q_row_norm.size == 64 and m0.k_row_norm.size == 32 and m0.q_row_norm.eps == 2e-6 and m0.bias.kind == "none" and not m0.sink
    assert (m2.window, m2.chunk, m2.softcap, m2.q_bias, m2.position.kind) == (37, None, 0.0, "", "none") and m2.q_row_norm.size == 24
    assert isinstance(m1, RglruSpec) and (m1.width, m1.blocks, m1.conv_taps, m1.decay_scale, m1.r_gate) == (48, 3, 3, 8.0, "l1.mix.ra")
    f0, f1 = spec.layers[0].ffn, spec.layers[1].ffn
    assert isinstance(f0, RoutedFfnSpec) and (f0.score, f0.group_top, f0.normalise, f0.route_scale, f0.n_identity) == ("sigmoid", 2, True, 1.0, 0)
    assert (f0.groups, f0.keep_groups, f0.top, f0.activation, f0.shared) == (3, 2, 2, "silu", None)
    assert isinstance(f1, GatedFfnSpec) and (f1.activation, f1.act_limit, f1.act_alpha) == ("swish_clamped", 1.2, 1.702)
    # the tensors the parts ask for are the ones the plain implementation draws, with its shapes
    needs = {n.name: tuple(n.shape) for n in tensor_needs(spec)}
    assert needs == P.tensor_shapes(sample())


@pytest.mark.parametrize("change, says", [
    (lambda c: c["layers"][1].__setitem__("type", "mamba"), "unknown layer type"),
    (lambda c: c["layers"][0]["mixer"].pop("vdim"), "'vdim' is missing"),
    (lambda c: c["layers"][0]["mixer"].__setitem__("kv_heads", 3), "not a multiple of kv_heads"),
    (lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 18), "at most dim"),
    (lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 5), "must be even"),
    (lambda c: c["layers"][0]["mixer"]["rot"]["scaling"].pop("original"), "'original' is missing"),
    (lambda c: c["layers"][0]["mixer"]["mask"].pop("size"), "'size' is missing"),
    (lambda c: c["layers"][1]["mixer"].__setitem__("blocks", 5), "not a multiple of blocks"),
    (lambda c: c["layers"][1]["mlp"].pop("limit"), "'limit' is missing"),
    (lambda c: c["layers"][0]["mlp"]["router"].__setitem__("top", 5), "exceeds the 4 experts"),
    (lambda c: c["layers"][0]["mlp"]["router"]["groups"].__setitem__("count", 4), "equal groups"),
    (lambda c: c["layers"][0]["mlp"].__setitem__("kind", "sparse"), "unknown kind"),
    (lambda c: c["loop"].__setitem__("stop", 5), "within the 4 layers"),
    (lambda c: c["loop"].__setitem__("times", 0), "'times' must be an integer >= 1"),
    (lambda c: c.__setitem__("streams", 0), "'streams' must be an integer >= 1"),
    (lambda c: c.pop("norm"), "'norm' must be an object"),
])
def test_errors_name_the_key(change, says):
    raw = copy.deepcopy(sample())
    change(raw)
    with pytest.raises(ConfigError) as e:
        DuperaxConfig.from_dict(raw)
    assert says in str(e.value)


def test_yarn_frequencies_by_hand():
    """Pairs that turn more than ``fast`` times within the original context keep their frequency, pairs that turn less
    than ``slow`` times are slowed down by the factor, those between are blended along a ramp."""
    rot = {"dims": 16, "base": 100.0, "scaling": {"factor": 4.0, "original": 200, "fast": 8.0, "slow": 1.0}}
    f, mag = P.yarn_frequencies(rot)
    plain = [100.0 ** (-2.0 * i / 16) for i in range(8)]
    turns = [200 * x / (2 * math.pi) for x in plain]
    assert abs(mag - (0.1 * math.log(4.0) + 1)) < 1e-12
    lo = max(math.floor(16 * math.log(200 / (2 * math.pi * 8.0)) / (2 * math.log(100.0))), 0)
    hi = min(math.ceil(16 * math.log(200 / (2 * math.pi * 1.0)) / (2 * math.log(100.0))), 15)
    assert (lo, hi) == (2, 7)
    for i in range(8):
        if i <= lo:
            assert float(f[i]) == plain[i] and turns[i] > 8.0 * 0.5
        elif i >= hi:
            assert abs(float(f[i]) - plain[i] / 4.0) < 1e-15
        else:
            assert plain[i] / 4.0 < float(f[i]) < plain[i]


def test_pages_of_chunks_that_are_over_come_back_and_every_run_has_its_memory():
    """The cache's bookkeeping alone (no device): a chunked group holds only the pages of the chunk a sequence is in; a
    layer that runs twice has two memories in one group; the recurrent runs have states of their own."""
    from agave_amd.cache import GroupKey, KVCache, StateNeed
    chunked = GroupKey(None, 2, 16, chunk=100, v_head_dim=8, layout="rows_vt")
    windowed = GroupKey(37, 3, 8, v_head_dim=24, layout="rows_vt")
    states = {m: {"S": StateNeed((48,), torch.float32), "conv": StateNeed((2, 48), torch.float32)} for m in (1, 3)}
    cache = KVCache({0: chunked, 2: windowed, 4: windowed}, states, 2, {chunked: 6, windowed: 6}, torch.float32, None, 1024)
    assert cache.group_of_memory[2] == cache.group_of_memory[4] != cache.group_of_memory[0]
    assert cache.index_in_group[2] != cache.index_in_group[4]
    g = cache.groups[cache.group_of_memory[0]]
    a = cache.alloc_slot()
    cache.plan_step([a], [99])
    cache.commit_step([a], [99])
    assert g.pool.n_free == 6 - 2                             # positions 0 .. 98: two pages
    pos0, plans = cache.plan_step([a], [1])
    assert plans[cache.group_of_memory[0]].base == [0]        # position 99 still sees its chunk's first page
    cache.commit_step([a], [1])
    assert g.pool.n_free == 6 - 1                             # the next query is at 100: the chunk from 100 on lives in page 1 only
    pos0, plans = cache.plan_step([a], [1])
    assert plans[cache.group_of_memory[0]].base == [1]
    cache.commit_step([a], [1])
    cache.plan_step([a], [250])                               # over two chunk borders in one step: pages 1 .. 5
    cache.commit_step([a], [250])
    assert cache.length(a) == 351 and g.pool.n_free == 6 - 2  # the chunk from 300 on: pages 4 and 5
    cache.free_slot(a)
    assert g.pool.n_free == 6 and cache.groups[cache.group_of_memory[2]].pool.n_free == 6
