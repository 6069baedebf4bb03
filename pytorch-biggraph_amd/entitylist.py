"""The entities of one side of a batch of edges, as ids.

Contract (torchbiggraph/entitylist.py:15-135): a 1-D int64 tensor of entity
offsets with list-like access -- an int gives a list of one, a slice must be
contiguous, an int64 tensor picks arbitrary positions -- plus concatenation,
comparison and device moves.  The reference pairs the ids with a ragged
TensorList for featurized entities; this path embeds by id only, so anything
that asks for the ragged half is refused with NotImplementedError.
"""
from typing import Any, Iterable

import torch

from .types import LongTensorType

_NO_FEATURES = "entities with features (a ragged TensorList) are outside the id-embedding path"


def _is_long(t: Any) -> bool:
    return isinstance(t, torch.Tensor) and t.dtype == torch.int64


def _checked_ids(ids: Any) -> LongTensorType:
    if not _is_long(ids):
        raise TypeError(f"entity ids are an int64 tensor, got {type(ids).__name__}"
                        + (f" of {ids.dtype}" if isinstance(ids, torch.Tensor) else ""))
    if ids.dim() != 1:
        raise ValueError(f"entity ids are one-dimensional, got shape {tuple(ids.shape)}")
    return ids


class EntityList:
    __slots__ = ("tensor",)

    def __init__(self, tensor: LongTensorType, tensor_list: Any = None) -> None:
        if tensor_list is not None:
            raise NotImplementedError(_NO_FEATURES)
        self.tensor = _checked_ids(tensor)

    # -- construction -------------------------------------------------------
    @classmethod
    def from_tensor(cls, tensor: LongTensorType) -> "EntityList":
        return cls(tensor)

    @classmethod
    def empty(cls) -> "EntityList":
        return cls(torch.zeros(0, dtype=torch.int64))

    @classmethod
    def cat(cls, entity_lists: Iterable["EntityList"]) -> "EntityList":
        return cls(torch.cat(tuple(part.tensor for part in entity_lists)))

    # -- views --------------------------------------------------------------
    def to_tensor(self) -> LongTensorType:
        return self.tensor

    def to_tensor_list(self):
        raise NotImplementedError(_NO_FEATURES)

    def to(self, *args, **kwargs) -> "EntityList":
        return EntityList(self.tensor.to(*args, **kwargs))

    def __len__(self) -> int:
        return int(self.tensor.numel())

    def __getitem__(self, index: Any) -> "EntityList":
        if isinstance(index, slice):
            if index.step not in (None, 1):
                raise ValueError(f"only contiguous slices are taken, got step {index.step}")
            picked = self.tensor[index]
        elif isinstance(index, int):
            picked = self.tensor.narrow(0, index if index >= 0 else index + len(self), 1)
        elif _is_long(index):
            picked = self.tensor[index]
        else:
            raise KeyError(f"cannot index entities with a {type(index).__name__}")
        return EntityList(picked)

    # -- comparison / display -------------------------------------------------
    def __eq__(self, other: Any) -> bool:
        if isinstance(other, EntityList):
            return torch.equal(self.tensor, other.tensor)
        return NotImplemented

    __hash__ = None

    def __repr__(self) -> str:
        return f"EntityList({self.tensor!r})"
