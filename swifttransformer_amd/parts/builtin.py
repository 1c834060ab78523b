"""Registration of the parts that ship with the engine."""
from .base import register_part
from .norm import LayerNorm, DynamicTanh
from .position import LearnedPositions, NoPositions, RotaryPositions
from .embedding import TokenEmbedding, LMHead
from .feed_forward import DenseFeedForward
from .attention import PagedAttention
from .arrangement import PreNorm, PostNorm, Sandwich
from .conv import CausalTokenConv
from .linear_attention import GatedLinearAttention
from .latent_attention import LatentAttention
from .routed import RoutedExperts
from .sink_attention import SinkAttention
from .state_space import Mamba2Mixer, GatedDeltaRule
from .reentry import InputInjection, AdditiveEntry
from .window_attention import GatedWindowAttention
from .retention import Retention
from .parallel import ParallelMixers
from .side_input import TokenSideInput

register_part("norm", "layer_norm", LayerNorm)
register_part("position", "learned", LearnedPositions)
register_part("position", "none", NoPositions)
register_part("embedding", "token", TokenEmbedding)
register_part("head", "linear", LMHead)
register_part("feed_forward", "dense", DenseFeedForward)
register_part("mixer", "paged_attention", PagedAttention)
register_part("arrangement", "pre_norm", PreNorm)
register_part("arrangement", "post_norm", PostNorm)
register_part("token_conv", "causal", CausalTokenConv)
register_part("mixer", "gated_linear_attention", GatedLinearAttention)
register_part("mixer", "latent_attention", LatentAttention)
register_part("feed_forward", "routed_experts", RoutedExperts)
register_part("position", "rotary", RotaryPositions)
register_part("mixer", "sink_attention", SinkAttention)
register_part("mixer", "mamba2", Mamba2Mixer)
register_part("mixer", "gated_delta", GatedDeltaRule)
register_part("reentry", "input_injection", InputInjection)
register_part("norm", "dynamic_tanh", DynamicTanh)
register_part("arrangement", "sandwich", Sandwich)
register_part("reentry", "additive", AdditiveEntry)
register_part("mixer", "gated_window_attention", GatedWindowAttention)
register_part("mixer", "retention", Retention)
register_part("mixer", "parallel", ParallelMixers)
register_part("side_input", "token_side", TokenSideInput)
from .arrangement import HyperConnections
from .embedding import HashedPairEmbedding
from .feed_forward import GatedFeedForward
from .tied_attention import TiedKeyValueAttention

register_part("arrangement", "hyper_connections", HyperConnections)
register_part("embedding", "hashed_pairs", HashedPairEmbedding)
register_part("feed_forward", "gated_dense", GatedFeedForward)
register_part("mixer", "tied_kv_attention", TiedKeyValueAttention)
