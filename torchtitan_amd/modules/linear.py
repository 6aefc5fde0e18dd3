"""``Linear``: the module whose weight the MXFP8 converter wraps.

Mirror of the reference's configurable linear (torchtitan/models/common/linear.py:14-56): an
``nn.Linear`` that also satisfies the ``Module`` protocol, built from a ``Config`` whose two
sizes arrive through ``build(in_features=..., out_features=...)``, initialised with a truncated
normal whose mean / std come from the config unless ``init_weights(init_std=...)`` overrides
the std.  The converter relies on the two private attributes ``_init_mean`` / ``_init_std``
surviving its ``__class__`` swap.
"""
from dataclasses import dataclass, field

import torch.nn as nn

from ..protocols import Module

_SIZE_FIELDS = ("in_features", "out_features")


class Linear(nn.Linear, Module):
    @dataclass(kw_only=True, slots=True)
    class Config(Module.Config):
        # sizes are not constructor arguments of the config: the parent model supplies them
        in_features: int = field(init=False)
        out_features: int = field(init=False)
        bias: bool = False
        init_mean: float = 0.0
        init_std: float = 0.02

    def __init__(self, config: Config):
        unset = [name for name in _SIZE_FIELDS if not hasattr(config, name)]
        if unset:
            raise TypeError(
                f"Linear.Config requires 'in_features' and 'out_features' to be set (missing: "
                f"{', '.join(unset)}): pass them to Config.build(...) or assign them on the Config "
                "instance before constructing Linear directly."
            )
        nn.Linear.__init__(self, config.in_features, config.out_features, bias=config.bias)
        self._init_mean, self._init_std = config.init_mean, config.init_std

    def init_weights(self, **kwargs) -> None:
        override = kwargs.pop("init_std", None)
        nn.init.trunc_normal_(self.weight, mean=self._init_mean,
                              std=self._init_std if override is None else override)
        if self.bias is not None:
            nn.init.zeros_(self.bias)
