"""The modules whose weights the MXFP8 converter wraps (host-side mirrors of the reference's)."""
from .linear import Linear
from .feed_forward import FeedForward, compute_ffn_hidden_dim
from .moe import GroupedExperts, MoE, TokenChoiceTopKRouter, TokenReorderer

__all__ = ["Linear", "FeedForward", "compute_ffn_hidden_dim", "GroupedExperts", "MoE",
           "TokenChoiceTopKRouter", "TokenReorderer"]
