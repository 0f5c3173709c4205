"""Typed configurations and the architecture registry."""
from .batasun import BatasunConfig
from .duperax import DuperaxConfig
from .errors import ConfigError, UnsupportedArchitecture
from .gemma3 import Gemma3Config
from .gusedra import GusedraConfig
from .registry import (Architecture, architectures, find_architecture, load_config,
                       read_config_json, register_architecture)
from .rilenex import RilenexConfig
from .spec import (RglruSpec, StreamMixSpec, AttentionSpec, BiasedAttentionSpec, LatentAttentionSpec, Mamba2Spec, RoutedFfnSpec, ScoreBiasSpec, DenseFfnSpec, FeedForwardSpec, GatedDeltaSpec, GatedFfnSpec, Hgrn2Spec, LayerSpec,
                   MixerSpec, ModelSpec, NormSpec, ParallelMixerSpec, PositionSpec, RunEntry, TalkingAttentionSpec)

register_architecture(Architecture(
    name=Gemma3Config.architecture,
    model_types=("gemma3_text", "gemma3"),          # aliases of src/arch.zig:22-24 that name this model
    parse=Gemma3Config.from_dict,
    spec=lambda cfg, names=None: cfg.model_spec(names)))

register_architecture(Architecture(
    name=RilenexConfig.architecture,
    model_types=("rilenex",),
    parse=RilenexConfig.from_dict,
    spec=lambda cfg, names=None: cfg.model_spec(names)))

register_architecture(Architecture(
    name=GusedraConfig.architecture,
    model_types=("gusedra",),
    parse=GusedraConfig.from_dict,
    spec=lambda cfg, names=None: cfg.model_spec(names)))

register_architecture(Architecture(
    name=BatasunConfig.architecture,
    model_types=("batasun",),
    parse=BatasunConfig.from_dict,
    spec=lambda cfg, names=None: cfg.model_spec(names)))

register_architecture(Architecture(
    name=DuperaxConfig.architecture,
    model_types=("duperax",),
    parse=DuperaxConfig.from_dict,
    spec=lambda cfg, names=None: cfg.model_spec(names)))

__all__ = [
    "DuperaxConfig", "RglruSpec", "StreamMixSpec", "ConfigError", "UnsupportedArchitecture", "Gemma3Config", "RilenexConfig", "GusedraConfig", "BatasunConfig", "LatentAttentionSpec", "Mamba2Spec", "BiasedAttentionSpec", "RoutedFfnSpec", "ScoreBiasSpec", "Architecture", "architectures",
    "find_architecture", "load_config", "read_config_json", "register_architecture",
    "AttentionSpec", "FeedForwardSpec", "GatedFfnSpec", "LayerSpec", "MixerSpec", "ModelSpec",
    "NormSpec", "PositionSpec", "RunEntry", "TalkingAttentionSpec", "GatedDeltaSpec", "Hgrn2Spec",
    "ParallelMixerSpec", "DenseFfnSpec"]
