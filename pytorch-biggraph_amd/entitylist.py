"""Lists of entities (reference: torchbiggraph/entitylist.py:15-135).

Only id-based entities are on the accelerated path; featurized entities
(TensorList) are not supported and `to_tensor_list` says so.
"""
from typing import Any, Sequence, Union

import torch

from .types import LongTensorType


def _is_long(t: Any) -> bool:
    return isinstance(t, torch.Tensor) and t.dtype == torch.int64


class EntityList:
    @classmethod
    def empty(cls) -> "EntityList":
        return cls(torch.empty((0,), dtype=torch.long))

    @classmethod
    def from_tensor(cls, tensor: LongTensorType) -> "EntityList":
        if tensor.dim() != 1:
            raise ValueError("Expected 1D tensor, got %dD" % tensor.dim())
        return cls(tensor)

    @classmethod
    def cat(cls, entity_lists: Sequence["EntityList"]) -> "EntityList":
        return cls(torch.cat([el.tensor for el in entity_lists]))

    def __init__(self, tensor: LongTensorType, tensor_list: Any = None) -> None:
        if not _is_long(tensor):
            raise TypeError("Expected long tensor as first argument, got %s" % type(tensor))
        if tensor_list is not None:
            raise NotImplementedError("Featurized entities (TensorList) are not supported")
        if tensor.dim() != 1:
            raise ValueError("Expected 1-dimensional tensor, got %d-dimensional one" % tensor.dim())
        self.tensor: LongTensorType = tensor

    def to_tensor(self) -> LongTensorType:
        return self.tensor

    def to_tensor_list(self):
        raise NotImplementedError("Featurized entities (TensorList) are not supported")

    def __eq__(self, other: Any) -> bool:
        if not isinstance(other, EntityList):
            return NotImplemented
        return torch.equal(self.tensor, other.tensor)

    def __repr__(self) -> str:
        return "EntityList(%r)" % (self.tensor,)

    __str__ = __repr__

    def __getitem__(self, index: Union[int, slice, LongTensorType]) -> "EntityList":
        if isinstance(index, int):
            return self[index:index + 1]
        if _is_long(index):
            return type(self)(self.tensor[index])
        if isinstance(index, slice):
            start, stop, step = index.indices(len(self))
            if step != 1:
                raise ValueError("Expected slice with step 1, got %d" % step)
            return type(self)(self.tensor[start:stop])
        raise KeyError("Unknown index type: %s" % type(index))

    def __len__(self) -> int:
        return self.tensor.shape[0]

    def to(self, *args, **kwargs) -> "EntityList":
        return type(self)(self.tensor.to(*args, **kwargs))
