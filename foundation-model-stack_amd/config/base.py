"""Typed model configurations that load from and save to JSON.

Behaviour follows the reference's ``ModelConfig`` (fms/utils/config.py:14-88):
``load`` ignores keys the dataclass does not have, ``updated`` returns a deep
copy with overrides and only logs unknown names, ``save`` writes ``as_dict``.
"""

from __future__ import annotations

import copy
import dataclasses
import json
import logging
import os
from typing import Type, TypeVar, Union

logger = logging.getLogger(__name__)

T = TypeVar("T", bound="ModelConfig")


@dataclasses.dataclass
class ModelConfig:
    @classmethod
    def load(cls: Type[T], json_file: Union[str, os.PathLike]) -> T:
        with open(json_file, "r", encoding="utf-8") as reader:
            return cls.from_dict(json.load(reader))

    @classmethod
    def from_dict(cls: Type[T], values: dict) -> T:
        """Keys that are no field of the dataclass are dropped (fms/utils/config.py:25-37)."""
        fields = {f.name: f for f in dataclasses.fields(cls)}
        kwargs = {}
        for key, value in values.items():
            if key not in fields:
                continue
            kind = fields[key].type
            if isinstance(kind, type) and issubclass(kind, ModelConfig) and isinstance(value, dict):
                value = kind.from_dict(value)
            kwargs[key] = value
        return cls(**kwargs)

    def as_dict(self) -> dict:
        return dataclasses.asdict(self)

    def save(self, file_path: Union[str, os.PathLike]) -> None:
        with open(file_path, "w", encoding="utf-8") as f:
            json.dump(self.as_dict(), f)

    def updated(self: T, **kwargs) -> T:
        """A deep copy with the named fields replaced (fms/utils/config.py:46-88).

        A dict given for a nested configuration updates that configuration.
        Names that are no field are logged, not raised.
        """
        clone = copy.deepcopy(self)
        unknown = []
        for key, value in kwargs.items():
            if not hasattr(clone, key):
                unknown.append(key)
                continue
            current = getattr(clone, key)
            if isinstance(current, ModelConfig) and isinstance(value, dict):
                setattr(clone, key, current.updated(**value))
            else:
                setattr(clone, key, value)
        if unknown:
            logger.info("Found the following unknown parameters while cloning and updating the configuration: %s", unknown)
        clone.validate()
        return clone

    def validate(self) -> None:
        """Subclasses raise ValueError for numbers that no model can be built from."""
