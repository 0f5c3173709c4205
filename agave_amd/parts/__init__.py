"""The parts a layer is put together from, and their registries."""
from .base import BuildEnv, Workspace, lookup, mixer_libraries, part_tensors, register, registered, state_tensor
from . import norm, position, attention, talking_attention, biased_attention, latent_attention, recurrent, rglru, parallel, ffn, routed_ffn, block, streams  # noqa: F401  (registers the built-in kinds)
from .attention import Attention
from .biased_attention import BiasedAttention
from .block import PostNormBlock, PreNormBlock, SandwichBlock, add_pending_and_norm
from .ffn import DenseFfn, GatedFfn
from .routed_ffn import RoutedFfn
from .parallel import ParallelMixer
from .latent_attention import LatentAttention
from .recurrent import GatedDelta, Hgrn2, Mamba2
from .rglru import Rglru
from .streams import StreamMix, StreamsBlock
from .short_conv import ShortConv
from .talking_attention import TalkingAttention
from .linear import Linear
from .norm import LayerNorm, Norm, NormedRows, RmsNorm, add_branch
from .position import NoPosition, RotaryPosition

__all__ = ["BuildEnv", "Workspace", "lookup", "mixer_libraries", "part_tensors", "register", "registered", "state_tensor",
           "Attention", "BiasedAttention", "GatedFfn", "DenseFfn", "RoutedFfn", "LayerNorm", "TalkingAttention", "GatedDelta", "Hgrn2", "Mamba2", "LatentAttention", "ParallelMixer", "ShortConv",
           "Rglru", "StreamMix", "StreamsBlock", "Linear", "Norm", "NormedRows", "RmsNorm", "add_branch", "RotaryPosition", "NoPosition", "SandwichBlock", "PreNormBlock", "PostNormBlock",
           "add_pending_and_norm"]
