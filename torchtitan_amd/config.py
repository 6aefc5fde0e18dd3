"""Config plumbing the converter plugs into: a class owns a nested ``Config`` dataclass and
``config.build(**kwargs)`` constructs the owner.

Mirrors the contract of the reference's ``Configurable`` (torchtitan/config/configurable.py:14-180)
as far as the MXFP8 path needs it: ``Config`` must be ``@dataclass(kw_only=True, slots=True)``;
``build()`` kwargs are either all config fields (absorbed into a copy of the config, conflicts
raise ``ValueError``) or all constructor arguments (forwarded); mixing raises ``TypeError``;
``field(init=False)`` slots must be filled by ``build()`` or pre-set.
"""
from __future__ import annotations

import dataclasses
from dataclasses import dataclass
from typing import ClassVar

import torch

_UNSET = "<UNSET>"


def _same(a, b) -> bool:
    if isinstance(a, torch.Tensor) or isinstance(b, torch.Tensor):
        return isinstance(a, torch.Tensor) and isinstance(b, torch.Tensor) and torch.equal(a, b)
    return a == b


class Configurable:
    @dataclass(kw_only=True, slots=True)
    class Config:
        _owner: ClassVar[type | None] = None

        def _get(self, name):
            try:
                return getattr(self, name)
            except AttributeError:
                return _UNSET

        def __repr__(self) -> str:
            body = ", ".join(
                f"{f.name}={_UNSET if self._get(f.name) is _UNSET else repr(self._get(f.name))}"
                for f in dataclasses.fields(self)
            )
            return f"{type(self).__name__}({body})"

        def to_dict(self) -> dict:
            out = {}
            for f in dataclasses.fields(self):
                v = self._get(f.name)
                if v is _UNSET:
                    continue
                if hasattr(v, "to_dict"):
                    v = v.to_dict()
                elif dataclasses.is_dataclass(v):
                    v = dataclasses.asdict(v)
                out[f.name] = v
            return out

        def _filled_copy(self, **late):
            """Copy with every ``init=False`` slot taken from `late` or from self."""
            twin = dataclasses.replace(self)
            for f in dataclasses.fields(self):
                if f.init:
                    continue
                if f.name in late:
                    setattr(twin, f.name, late[f.name])
                elif self._get(f.name) is not _UNSET:
                    setattr(twin, f.name, getattr(self, f.name))
                else:
                    raise TypeError(
                        f"{type(self).__name__} field '{f.name}' (init=False) was not provided via build()"
                    )
            return twin

        def build(self, **kwargs):
            owner = type(self)._owner
            if owner is None:
                raise NotImplementedError(
                    f"{type(self).__name__} has no owner class. Define Config inside a Configurable subclass."
                )
            names = {f.name for f in dataclasses.fields(self)}
            as_fields = {k for k in kwargs if k in names}
            as_ctor = set(kwargs) - as_fields
            if as_fields and as_ctor:
                raise TypeError(
                    f"{type(self).__name__}.build() kwargs must either all be config fields or all be "
                    f"constructor arguments. Got config fields {as_fields} mixed with non-config fields {as_ctor}."
                )
            if as_fields:
                for k in as_fields:
                    cur = self._get(k)
                    if cur is not _UNSET and not _same(cur, kwargs[k]):
                        raise ValueError(
                            f"{type(self).__name__}.build() conflict for '{k}': config has {cur!r} but got {kwargs[k]!r}"
                        )
                return owner(config=self._filled_copy(**kwargs))
            return owner(config=self._filled_copy(), **kwargs)

    def __init_subclass__(cls, **kwargs):
        super().__init_subclass__(**kwargs)
        cfg = cls.__dict__.get("Config")
        if cfg is None or not issubclass(cfg, Configurable.Config):
            return
        if "__slots__" not in cfg.__dict__:
            raise TypeError(f"{cls.__name__}.Config must use @dataclass(kw_only=True, slots=True)")
        for f in dataclasses.fields(cfg):
            if f.init and not f.kw_only:
                raise TypeError(f"{cls.__name__}.Config field '{f.name}' must be keyword-only")
        cfg.__repr__ = Configurable.Config.__repr__
        cfg._owner = cls
