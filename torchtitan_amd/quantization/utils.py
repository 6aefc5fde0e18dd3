"""Shared module filter of the low-precision converters
(torchtitan/components/quantization/utils.py:10-27)."""
import torch.nn as nn


def module_filter_fn(mod: nn.Module, fqn: str, filter_fqns: list[str]) -> bool:
    """True for an ``nn.Linear`` whose two weight dimensions are multiples of 16 and whose
    fully qualified name contains none of `filter_fqns`."""
    if not isinstance(mod, nn.Linear):
        return False
    rows, cols = mod.weight.shape
    if rows % 16 or cols % 16:
        return False
    return not any(part in fqn for part in filter_fqns)
