"""Plugin protocols the trainer drives: ``Module`` and the model-converter container.

Counterparts of torchtitan/protocols/module.py:12-23 and
torchtitan/protocols/model_converter.py:17-101.
"""
from __future__ import annotations

import logging
from dataclasses import dataclass, field
from typing import Any, Protocol

import torch.nn as nn

from .config import Configurable

logger = logging.getLogger("torchtitan_amd")


class Module(nn.Module, Configurable):
    """nn.Module that is also Configurable; ``init_weights`` defaults to a no-op."""

    def init_weights(self, **kwargs) -> None:
        return None


class ModelConverter(Protocol):
    """Something that rewrites a model in place, with an optional post-optimizer callback."""

    def convert(self, model: nn.Module): ...

    def post_optimizer_hook(self, model: nn.Module | list[nn.Module]): ...


def _validate_quantization(converter_configs: list) -> None:
    """All quantization converters in one container must share one ``_quantization_type``."""
    from .quantization import QuantizationConverter

    seen: str | None = None
    for cc in converter_configs:
        if not isinstance(cc, QuantizationConverter.Config):
            continue
        kind = cc._quantization_type
        if seen is None:
            seen = kind
        assert kind == seen, (
            f"Cannot combine model converters with different quantization types: '{kind}' and '{seen}'"
        )


class ModelConvertersContainer(Configurable):
    """Builds each converter from its Config and applies them in order."""

    @dataclass(kw_only=True, slots=True)
    class Config(Configurable.Config):
        converters: list = field(default_factory=list)
        print_after_conversion: bool = False

    def __init__(self, config: Config, *, parallel_dims: Any, model_compile_enabled: bool):
        _validate_quantization(config.converters)
        self.converters = [
            cc.build(parallel_dims=parallel_dims, model_compile_enabled=model_compile_enabled)
            for cc in config.converters
        ]
        self.print_after_conversion = config.print_after_conversion

    def convert(self, model: nn.Module):
        for conv in self.converters:
            conv.convert(model)
        if self.print_after_conversion:
            logger.info("Model definition after conversion:\n\n%s\n\n", model)

    def post_optimizer_hook(self, model: nn.Module | list[nn.Module]):
        for conv in self.converters:
            conv.post_optimizer_hook(model)
