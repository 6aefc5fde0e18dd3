"""Quantization converters (torchtitan/components/quantization/__init__.py:22-36)."""
from dataclasses import dataclass
from typing import ClassVar

from ..config import Configurable


class QuantizationConverter(Configurable):
    """Base of every quantization converter; lets containers recognise them by isinstance."""

    @dataclass(kw_only=True, slots=True)
    class Config(Configurable.Config):
        _quantization_type: ClassVar[str]


FP8_GROUP_ALIGNMENT_SIZE = 16
MXFP8_GROUP_ALIGNMENT_SIZE = 32
