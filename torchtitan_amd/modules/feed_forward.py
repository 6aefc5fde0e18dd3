"""SwiGLU feed-forward ``w2(silu(w1 x) * w3 x)`` (torchtitan/models/common/feed_forward.py:18-67)."""
from dataclasses import dataclass, field

import torch
import torch.nn.functional as F

from ..mx_blocks import feed_forward_fusable, mx_feed_forward, mx_swiglu_linear, swiglu_fusable
from ..protocols import Module
from .linear import Linear


def compute_ffn_hidden_dim(dim: int, *, multiple_of: int = 1,
                           ffn_dim_multiplier: float | None = None) -> int:
    """2/3 * 4 * dim, optional multiplier, rounded up to `multiple_of` (Llama-3 8B: 14336)."""
    hidden = int(2 * 4 * dim / 3)
    if ffn_dim_multiplier is not None:
        hidden = int(ffn_dim_multiplier * hidden)
    return -(-hidden // multiple_of) * multiple_of


class FeedForward(Module):
    @dataclass(kw_only=True, slots=True)
    class Config(Module.Config):
        hidden_dim: int
        linear_bias: bool = False
        dim: int = field(init=False)

    def __init__(self, config: Config):
        super().__init__()
        lin = Linear.Config(bias=config.linear_bias)
        self.w1 = lin.build(in_features=config.dim, out_features=config.hidden_dim)
        self.w2 = lin.build(in_features=config.hidden_dim, out_features=config.dim)
        self.w3 = lin.build(in_features=config.dim, out_features=config.hidden_dim)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if (self.w1.bias is None and self.w3.bias is None
                and feed_forward_fusable(x, self.w1.weight, self.w2.weight, self.w3.weight)):
            # all three converted: gate and its backward inside the MXFP8 cast kernels
            return mx_feed_forward(x, self.w1.weight, self.w2.weight, self.w3.weight, self.w2.bias)
        h1, h3 = self.w1(x), self.w3(x)
        if swiglu_fusable(h1, h3, self.w2.weight):  # converted w2: gate inside the MXFP8 cast
            return mx_swiglu_linear(h1, h3, self.w2.weight, self.w2.bias)
        return self.w2(F.silu(h1) * h3)

    def init_weights(self, init_std: float = 0.02, **kwargs):
        self.w1.init_weights()
        self.w2.init_weights(init_std=init_std)
        self.w3.init_weights(init_std=init_std)
