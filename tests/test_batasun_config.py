"""The Batasun configuration without a GPU: parser, round trip, errors that name the key, the spec and its run
order, the tensors the parts ask for, and the cache bookkeeping of latent rows that two layers share."""
import copy

import pytest
import torch

import plain_batasun as P
from agave_amd.config import BatasunConfig, ConfigError, find_architecture
from agave_amd.config.spec import LatentAttentionSpec, Mamba2Spec, RoutedFfnSpec
from agave_amd.engine.model import tensor_needs


def sample():
    return P.config([
        P.mamba_layer(4, 12, 8, 2, 4, 3, mlp=P.moe(5, 2, 24, 1.25, shared_ff=16, shared_limit=3.0)),
        P.latent_layer(3, 16, 8, 20, 24, 40, base=5000.0, mlp=None),
        P.mamba_layer(2, 6, 16, 1, 1, 1),
        P.latent_layer(5, 8, 8, 4, 12, 40, base=5000.0, kv_from=1, mlp=P.moe(3, 3, 8, 0.5)),
        P.latent_layer(2, 8, 8, 4, 12, 40, base=5000.0, kv_from=1)], vocab=71, width=40, eps=2e-6)


def test_found_by_its_name_and_round_trip():
    raw = sample()
    arch = find_architecture(raw)
    assert arch.name == "Batasun"
    cfg = arch.parse(raw)
    assert isinstance(cfg, BatasunConfig) and cfg.to_dict() == raw
    assert BatasunConfig.from_dict(cfg.to_dict()) == cfg
    assert cfg.layers[1].mixer.kv_rank == 40 and cfg.layers[3].mixer.kv_from == 1 and cfg.layers[0].mlp.shared_limit == 3.0
    assert cfg.layers[2].mlp is None and cfg.layers[3].mlp.shared_ff is None


def test_spec_says_everything_the_parts_need():
    cfg = BatasunConfig.from_dict(sample())
    spec = cfg.model_spec()
    assert [(e.layer, e.memory, e.writes) for e in spec.order] == [(0, 0, True), (1, 1, True), (2, 2, True), (3, 1, False), (4, 1, False)]
    assert spec.embed_norm is not None and spec.embed_norm.add_one and spec.final_norm.add_one and spec.embed_scale == 1.0
    assert all(l.kind == "postnorm" and l.pre_mixer_norm is None and l.pre_ffn_norm is None for l in spec.layers)
    m0, m1, m3 = spec.layers[0].mixer, spec.layers[1].mixer, spec.layers[3].mixer
    assert isinstance(m0, Mamba2Spec) and (m0.n_heads, m0.v_head_dim, m0.state, m0.groups, m0.conv_taps, m0.norm_groups) == (4, 12, 8, 2, 4, 3)
    assert isinstance(m1, LatentAttentionSpec) and m1.kv_down == "l1.mix.dkv" and m1.position.theta == 5000.0 and m1.position.rotary_dim == 8
    assert m3.kv_down == "" and m3.kv_norm == "" and m3.k_up == "l3.mix.uk" and m3.norm_eps == 2e-6
    f0, f3 = spec.layers[0].ffn, spec.layers[3].ffn
    assert isinstance(f0, RoutedFfnSpec) and f0.score == "softmax_top" and f0.correction == "l0.mlp.router.b" and f0.act_limit == 1.25
    assert f0.shared.act_limit == 3.0 and f0.shared_gate == "l0.mlp.shared.sg" and f0.act_alpha == 1.702 and f0.activation == "swish_clamped"
    assert f3.shared is None and f3.shared_gate == "" and f3.top == 3 and spec.layers[1].ffn is None and spec.layers[1].post_ffn_norm is None
    # the tensors the parts ask for are the ones the plain implementation draws, with its shapes
    needs = {n.name: tuple(n.shape) for n in tensor_needs(spec)}
    assert needs == P.tensor_shapes(sample())


@pytest.mark.parametrize("change, says", [
    (lambda c: c["layers"][1].__setitem__("type", "attention"), "unknown layer type"),
    (lambda c: c["layers"][1]["mixer"].pop("kv_rank"), "'kv_rank' is missing"),
    (lambda c: c["layers"][1]["mixer"]["rot"].__setitem__("dims", 10), "at most rot_dim"),
    (lambda c: c["layers"][1]["mixer"]["rot"].__setitem__("dims", 5), "must be even"),
    (lambda c: c["layers"][3]["mixer"].__setitem__("kv_from", 3), "earlier layer"),
    (lambda c: c["layers"][3]["mixer"].__setitem__("kv_from", 0), "without a latent projection"),
    (lambda c: c["layers"][4]["mixer"].__setitem__("kv_from", 3), "without a latent projection"),
    (lambda c: c["layers"][3]["mixer"].__setitem__("kv_rank", 32), "must equal those of layer 1"),
    (lambda c: c["layers"][3]["mixer"]["rot"].__setitem__("base", 7.0), "must equal those of layer 1"),
    (lambda c: c["layers"][0]["mixer"].__setitem__("groups", 3), "not a multiple of groups"),
    (lambda c: c["layers"][0]["mixer"].__setitem__("norm_groups", 5), "equal parts"),
    (lambda c: c["layers"][0]["mlp"]["router"].__setitem__("top", 6), "exceeds the 5 experts"),
    (lambda c: c["layers"][0]["mlp"]["expert"].pop("limit"), "'limit' is missing"),
    (lambda c: c["layers"][0]["mlp"].__setitem__("kind", "dense"), "unknown kind"),
    (lambda c: c.pop("norm"), "'norm' must be an object"),
])
def test_errors_name_the_key(change, says):
    raw = copy.deepcopy(sample())
    change(raw)
    with pytest.raises(ConfigError) as e:
        BatasunConfig.from_dict(raw)
    assert says in str(e.value)


def test_readers_share_the_latent_rows_of_their_source():
    """The cache's bookkeeping alone (no device): one memory of latent rows for layers 1, 3 and 4, of one key head
    whose rows hold the latent and the rotated part; states for the two recurrent layers."""
    from agave_amd.cache import GroupKey, KVCache, StateNeed
    key = GroupKey(None, 1, 48, v_head_dim=40, layout="rows_vt")
    states = {0: {"S": StateNeed((4, 12, 8), torch.float32), "conv": StateNeed((3, 80), torch.float32)},
              2: {"S": StateNeed((2, 6, 16), torch.float32), "conv": StateNeed((0, 44), torch.float32)}}
    cache = KVCache({1: key}, states, 2, {key: 6}, torch.float32, None, 256)
    a, b = cache.alloc_slot(), cache.alloc_slot()
    cache.plan_step([a, b], [130, 64])
    cache.commit_step([a, b], [130, 64])
    pool = cache.groups[0].pool
    assert pool.n_free == 6 - 3 - 1
    cache.plan_step([a], [62])                                # to 192: still three pages
    cache.commit_step([a], [62])
    assert pool.n_free == 2
    with pytest.raises(Exception):
        cache.plan_step([a, b], [1, 129])                     # four and four pages do not fit six
    cache.free_slot(a)
    assert pool.n_free == 5
    c = cache.alloc_slot()                                    # the freed slot and its pages are used again
    assert c == a
    cache.plan_step([c], [200])
    cache.commit_step([c], [200])
    assert pool.n_free == 1
    cache.free_slot(b)
    cache.free_slot(c)
    assert pool.n_free == 6
