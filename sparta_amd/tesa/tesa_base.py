"""Abstract interfaces of a sparsity-attribute index and of the object that builds
it (sparta/tesa/tesa_base.py)."""
from __future__ import annotations

import abc
from typing import Any

import torch


class TeSAIndexes(abc.ABC):
    """Index tensors describing where the live part of a masked tensor sits."""

    def __init__(self, function_context: 'TeSAFunctionContext', mask: torch.Tensor):
        self.function_context = function_context
        self.raw_mask = mask
        self.device = mask.device

    @abc.abstractmethod
    def get_mask(self) -> torch.Tensor:
        """The element mask actually covered by the index."""

    def to(self, device: Any) -> 'TeSAIndexes':
        """Move every tensor attribute to `device` (sparta/tesa/tesa_base.py:23-27; the
        reference discards the moved copies and only updates `device`, here the
        attributes are rebound).  Cached host-side values survive the move."""
        self.device = torch.device(device)
        for name, value in list(self.__dict__.items()):
            if isinstance(value, torch.Tensor):
                setattr(self, name, value.to(device))
            elif isinstance(value, dict):
                for key, item in value.items():
                    if isinstance(item, torch.Tensor):
                        value[key] = item.to(device)
        return self


class TeSAFunctionContext(abc.ABC):
    """Builds indexes for one sparsity format and converts values."""

    @abc.abstractmethod
    def build_indexes(self, mask: torch.Tensor, *args) -> TeSAIndexes:
        ...

    @abc.abstractmethod
    def convert(self, dense: torch.Tensor, *args) -> torch.Tensor:
        ...

    @abc.abstractmethod
    def inverse(self, sparse_val: torch.Tensor, *args) -> torch.Tensor:
        ...
