"""Lists of edges (reference: torchbiggraph/edgelist.py:15-179): two entity
lists, a relation that is a scalar (one type for all edges) or a vector (one per
edge), and optional per-edge weights."""
from typing import Any, Optional, Sequence, Union

import torch

from .entitylist import EntityList, _is_long
from .types import FloatTensorType, LongTensorType


class EdgeList:
    @classmethod
    def empty(cls) -> "EdgeList":
        return cls(EntityList.empty(), EntityList.empty(), torch.empty((0,), dtype=torch.long))

    @classmethod
    def cat(cls, edge_lists: Sequence["EdgeList"]) -> "EdgeList":
        lhs = EntityList.cat([el.lhs for el in edge_lists])
        rhs = EntityList.cat([el.rhs for el in edge_lists])
        weighted = [el.has_weight() for el in edge_lists]
        if any(weighted):
            if not all(weighted):
                raise RuntimeError("Can't concatenate edgelists with and without weight field.")
            weight = torch.cat([el.weight.expand((len(el),)) for el in edge_lists])
        else:
            weight = None
        if all(el.has_scalar_relation_type() for el in edge_lists):
            kinds = {el.get_relation_type_as_scalar() for el in edge_lists}
            if len(kinds) == 1:
                (kind,) = kinds
                return cls(lhs, rhs, torch.tensor(kind, dtype=torch.long), weight)
        rel = torch.cat([el.rel.expand((len(el),)) for el in edge_lists])
        return cls(lhs, rhs, rel, weight)

    def __init__(self, lhs: EntityList, rhs: EntityList, rel: LongTensorType,
                 weight: Optional[FloatTensorType] = None) -> None:
        if not isinstance(lhs, EntityList) or not isinstance(rhs, EntityList):
            raise TypeError(
                "Expected left- and right-hand side to be entity lists, got %s and %s instead" % (type(lhs), type(rhs))
            )
        if not _is_long(rel):
            raise TypeError("Expected relation to be a long tensor, got %s" % type(rel))
        if len(lhs) != len(rhs):
            raise ValueError(
                "The left- and right-hand side entity lists have different lengths: %d != %d" % (len(lhs), len(rhs))
            )
        if rel.dim() > 1:
            raise ValueError(
                "The relation can be either a scalar or a 1-dimensional tensor, got a %d-dimensional tensor" % rel.dim()
            )
        if rel.dim() == 1 and rel.shape[0] != len(lhs):
            raise ValueError(
                "The relation has a different length than the entity lists: %d != %d" % (rel.shape[0], len(lhs))
            )
        if weight is not None and weight.nelement() == 0:
            weight = None
        if weight is not None:
            if weight.dim() > 1:
                raise ValueError(
                    "The weight can be either a scalar or a 1-dimensional tensor, got a %d-dimensional tensor"
                    % weight.dim()
                )
            if weight.dim() == 1 and weight.shape[0] != len(lhs):
                raise ValueError(
                    "The weight has a different length than the entity lists: %d != %d" % (weight.shape[0], len(lhs))
                )
        self.lhs = lhs
        self.rhs = rhs
        self.rel = rel
        self.weight = weight

    def has_scalar_relation_type(self) -> bool:
        return self.rel.dim() == 0

    def get_relation_type_as_scalar(self) -> int:
        if self.rel.dim() != 0:
            raise RuntimeError("The relation isn't a scalar")
        return int(self.rel)

    def get_relation_type_as_vector(self) -> LongTensorType:
        if self.rel.dim() == 0:
            return self.rel.view((1,)).expand((len(self),))
        return self.rel

    def get_relation_type(self) -> Union[int, LongTensorType]:
        if self.has_scalar_relation_type():
            return self.get_relation_type_as_scalar()
        return self.get_relation_type_as_vector()

    def has_weight(self) -> bool:
        return self.weight is not None

    def get_weight(self) -> Union[float, torch.Tensor]:
        return self.weight if self.has_weight() else 1

    def __eq__(self, other: Any) -> bool:
        if not isinstance(other, EdgeList):
            return NotImplemented
        return self.lhs == other.lhs and self.rhs == other.rhs and torch.equal(self.rel, other.rel)

    def __repr__(self) -> str:
        return "EdgeList(%r, %r, %r, %r)" % (self.lhs, self.rhs, self.rel, self.weight)

    __str__ = __repr__

    def __getitem__(self, index: Union[int, slice, LongTensorType]) -> "EdgeList":
        if not isinstance(index, (int, slice)) and not _is_long(index):
            raise TypeError("Index can only be int, slice or long tensor, got %s" % type(index))
        if _is_long(index) and index.dim() != 1:
            raise ValueError("Long tensor index must be 1-dimensional, got %d-dimensional" % (index.dim(),))
        rel = self.rel if self.has_scalar_relation_type() else self.rel[index]
        weight = self.weight[index] if self.has_weight() else None
        return type(self)(self.lhs[index], self.rhs[index], rel, weight)

    def __len__(self) -> int:
        return len(self.lhs)

    def to(self, *args, **kwargs) -> "EdgeList":
        weight = self.weight.to(*args, **kwargs) if self.weight is not None else None
        return type(self)(self.lhs.to(*args, **kwargs), self.rhs.to(*args, **kwargs), self.rel.to(*args, **kwargs), weight)
