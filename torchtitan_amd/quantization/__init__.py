"""Quantization converters: the shared base class and the group-alignment constants
(torchtitan/components/quantization/__init__.py:22-36)."""
from dataclasses import dataclass
from typing import ClassVar

from ..config import Configurable

# Token groups of a grouped GEMM are padded to these many rows: 32 is one MX scaling block
# along the token axis (what the wgrad's column-wise cast needs), 16 the float8 row-wise rule.
MXFP8_GROUP_ALIGNMENT_SIZE = 32
FP8_GROUP_ALIGNMENT_SIZE = 16


class QuantizationConverter(Configurable):
    """What every quantization converter derives from, so that a container of converters can
    tell them from other converters with isinstance and refuse a mix of quantization types."""

    @dataclass(kw_only=True, slots=True)
    class Config(Configurable.Config):
        # name of the number format ("mxfp8", "float8", ...); one per converter class
        _quantization_type: ClassVar[str]


def quantization_type_of(config) -> str | None:
    """The `_quantization_type` of a converter config, None for a config of another kind."""
    return getattr(config, "_quantization_type", None) if isinstance(config, QuantizationConverter.Config) else None
