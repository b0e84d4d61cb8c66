"""A minimal `Configurable` in the shape the kernel classes need.

AXLearn kernel classes are built as `cls.default_config().set(**kwargs).instantiate()`
(axlearn/common/flash_attention/utils.py:154). This module supplies just that protocol; it is not a
re-implementation of axlearn/common/config.py.
"""

from __future__ import annotations

import copy
import dataclasses
from typing import Any, Optional


def config_class(cls):
    """Marks a nested `Config` class; fields become dataclass fields."""
    return dataclasses.dataclass(cls)


class Configurable:
    @config_class
    class Config:
        klass: Optional[type] = None

        def set(self, **kwargs) -> "Configurable.Config":
            for name, value in kwargs.items():
                if not any(f.name == name for f in dataclasses.fields(self)):
                    raise AttributeError(f"{type(self).__qualname__} has no field {name!r}")
                setattr(self, name, value)
            return self

        def clone(self, **kwargs) -> "Configurable.Config":
            return copy.deepcopy(self).set(**kwargs)

        def instantiate(self, **kwargs) -> Any:
            return self.klass(self, **kwargs)

    @classmethod
    def default_config(cls) -> "Configurable.Config":
        return cls.Config(klass=cls)

    def __init__(self, cfg: "Configurable.Config"):
        self._config = copy.deepcopy(cfg)

    @property
    def config(self) -> "Configurable.Config":
        return copy.deepcopy(self._config)
