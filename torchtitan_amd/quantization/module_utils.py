"""Keep the ``Module`` protocol (and ``_init_mean`` / ``_init_std``) alive across a conversion
that swaps module classes.  Behaviour of torchtitan/components/quantization/module_utils.py:21-118.
"""
from __future__ import annotations

from typing import Any

import torch.nn as nn

from ..protocols import Module


def capture_module_attrs(model: nn.Module, attr_names: list[str],
                         nn_module_cls: type[nn.Module] = nn.Linear) -> dict[str, dict[str, Any]]:
    """{fqn: {attr: value}} for every `nn_module_cls` instance that has all of `attr_names`."""
    saved: dict[str, dict[str, Any]] = {}
    for fqn, mod in model.named_modules():
        if not isinstance(mod, nn_module_cls):
            continue
        if any(not hasattr(mod, a) for a in attr_names):
            continue
        saved[fqn] = {a: getattr(mod, a) for a in attr_names}
    return saved


def _refuse_construction(self, *args, **kwargs):
    raise RuntimeError(
        f"{type(self).__name__} is a patched class created by inject_module_protocol "
        "and should not be constructed directly."
    )


def inject_module_protocol(model: nn.Module, module_cls: type[Module],
                           saved_attrs: dict[str, dict[str, Any]] | None = None,
                           nn_module_cls: type[nn.Module] = nn.Linear) -> None:
    """Give every `nn_module_cls` instance that lost the ``Module`` protocol a synthetic class
    deriving from (its current class, `module_cls`), one per original class, and restore attrs."""
    synthetic: dict[type, type] = {}
    for fqn, mod in model.named_modules():
        if not isinstance(mod, nn_module_cls) or isinstance(mod, Module):
            continue
        current = type(mod)
        patched = synthetic.get(current)
        if patched is None:
            patched = type(f"{current.__name__}_With{module_cls.__name__}", (current, module_cls),
                           {"__init__": _refuse_construction})
            synthetic[current] = patched
        mod.__class__ = patched
        for name, value in (saved_attrs or {}).get(fqn, {}).items():
            setattr(mod, name, value)


def verify_module_protocol(model: nn.Module, target_cls: type[nn.Module],
                           module_cls: type[Module] = Module) -> None:
    """Raise RuntimeError naming every `target_cls` instance that is not a `module_cls`."""
    offenders = [
        f"'{fqn}' ({type(mod).__name__})"
        for fqn, mod in model.named_modules()
        if isinstance(mod, target_cls) and not isinstance(mod, module_cls)
    ]
    if offenders:
        raise RuntimeError(
            f"The following {target_cls.__name__} modules do not satisfy "
            f"{module_cls.__name__} protocol: {', '.join(offenders)}"
        )
