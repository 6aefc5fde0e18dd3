"""``Linear``: nn.Linear + Module protocol with truncated-normal init
(torchtitan/models/common/linear.py:14-56)."""
from dataclasses import dataclass, field

import torch.nn as nn

from ..protocols import Module


class Linear(nn.Linear, Module):
    @dataclass(kw_only=True, slots=True)
    class Config(Module.Config):
        in_features: int = field(init=False)
        out_features: int = field(init=False)
        bias: bool = False
        init_mean: float = 0.0
        init_std: float = 0.02

    def __init__(self, config: Config):
        missing = [n for n in ("in_features", "out_features") if not hasattr(config, n)]
        if missing:
            raise TypeError(
                "Linear.Config requires 'in_features' and 'out_features' to be set. "
                "Use Config.build(in_features=..., out_features=...) or set them "
                "on the Config instance before constructing Linear directly."
            )
        super().__init__(config.in_features, config.out_features, bias=config.bias)
        self._init_mean = config.init_mean
        self._init_std = config.init_std

    def init_weights(self, **kwargs) -> None:
        std = kwargs.pop("init_std", None)
        nn.init.trunc_normal_(self.weight, mean=self._init_mean,
                              std=self._init_std if std is None else std)
        if self.bias is not None:
            nn.init.zeros_(self.bias)
