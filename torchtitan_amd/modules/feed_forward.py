"""SwiGLU feed-forward block ``w2(silu(w1 x) * w3 x)``.

Mirror of the reference's shared block (torchtitan/models/common/feed_forward.py:18-67): the
config carries the final hidden size, the model size arrives through ``build(dim=...)``, and the
three projections are ``Linear`` modules named w1 (gate), w3 (up) and w2 (down) so that the
converter's FQN filters and checkpoints line up.  When the converter has wrapped the weights,
``forward`` hands the block to the fused MXFP8 functions instead of three separate linears.
"""
from dataclasses import dataclass, field

import torch
import torch.nn.functional as F

from ..mx_blocks import feed_forward_fusable, mx_feed_forward, mx_swiglu_linear, swiglu_fusable
from ..protocols import Module
from .linear import Linear


def compute_ffn_hidden_dim(dim: int, *, multiple_of: int = 1,
                           ffn_dim_multiplier: float | None = None) -> int:
    """Hidden size of a Llama-style SwiGLU block: two thirds of 4 * dim, times the optional
    multiplier, rounded up to a multiple of `multiple_of` (dim 4096, multiplier 1.3, multiple
    1024 -> 14336)."""
    hidden = int(8 * dim / 3)
    if ffn_dim_multiplier is not None:
        hidden = int(ffn_dim_multiplier * hidden)
    return -(-hidden // multiple_of) * multiple_of


class FeedForward(Module):
    @dataclass(kw_only=True, slots=True)
    class Config(Module.Config):
        hidden_dim: int
        linear_bias: bool = False
        dim: int = field(init=False)  # supplied by build(dim=...)

    def __init__(self, config: Config):
        super().__init__()
        make = Linear.Config(bias=config.linear_bias).build
        up = dict(in_features=config.dim, out_features=config.hidden_dim)
        self.w1 = make(**up)
        self.w2 = make(in_features=config.hidden_dim, out_features=config.dim)
        self.w3 = make(**up)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        w1, w2, w3 = self.w1, self.w2, self.w3
        if w1.bias is None and w3.bias is None and feed_forward_fusable(x, w1.weight, w2.weight, w3.weight):
            # all three converted: gate and its backward inside the MXFP8 cast kernels
            return mx_feed_forward(x, w1.weight, w2.weight, w3.weight, w2.bias)
        gate, up = w1(x), w3(x)
        if swiglu_fusable(gate, up, w2.weight):  # converted w2 only: gate inside the cast feeding it
            return mx_swiglu_linear(gate, up, w2.weight, w2.bias)
        return w2(F.silu(gate) * up)

    def init_weights(self, init_std: float = 0.02, **kwargs):
        # the down projection takes the depth-scaled std, gate and up their configured default
        for proj, std in ((self.w1, None), (self.w2, init_std), (self.w3, init_std)):
            proj.init_weights(**({} if std is None else {"init_std": std}))
