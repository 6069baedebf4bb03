"""The edges handed to the model: a left and a right EntityList of equal length, a
relation that is either 0-dimensional (one type for every edge: the standard,
single-relation batch) or one entry per edge (dynamic relations), and an optional
weight per edge.  Contract: torchbiggraph/edgelist.py:15-179."""
from typing import Any, Optional, Sequence, Union

import torch

from .entitylist import EntityList, _is_long
from .types import FloatTensorType, LongTensorType


def _per_edge_or_scalar(what: str, t: torch.Tensor, num_edges: int) -> None:
    """`t` is 0-dimensional or holds one entry per edge."""
    if t.dim() > 1:
        raise ValueError(f"the {what} is a scalar or a vector, not a {t.dim()}-dimensional tensor")
    if t.dim() == 1 and t.shape[0] != num_edges:
        raise ValueError(f"the {what} has {t.shape[0]} entries for {num_edges} edges")


class EdgeList:
    def __init__(self, lhs: EntityList, rhs: EntityList, rel: LongTensorType,
                 weight: Optional[FloatTensorType] = None) -> None:
        for side in (lhs, rhs):
            if not isinstance(side, EntityList):
                raise TypeError(f"both sides of an EdgeList are EntityLists, got {type(side).__name__}")
        if not _is_long(rel):
            raise TypeError(f"the relation is an int64 tensor, got {type(rel).__name__}")
        if len(lhs) != len(rhs):
            raise ValueError(f"{len(lhs)} left-hand entities for {len(rhs)} right-hand entities")
        _per_edge_or_scalar("relation", rel, len(lhs))
        if weight is not None and weight.nelement() == 0:
            weight = None  # an empty weight tensor means "unweighted"
        if weight is not None:
            _per_edge_or_scalar("weight", weight, len(lhs))
        self.lhs, self.rhs, self.rel, self.weight = lhs, rhs, rel, weight

    @classmethod
    def empty(cls) -> "EdgeList":
        return cls(EntityList.empty(), EntityList.empty(), torch.empty((0,), dtype=torch.long))

    @classmethod
    def cat(cls, edge_lists: Sequence["EdgeList"]) -> "EdgeList":
        """Concatenation.  The result keeps a scalar relation only when every part has
        the same scalar; weighted and unweighted parts do not mix."""
        parts = list(edge_lists)
        weighted = sum(p.has_weight() for p in parts)
        if 0 < weighted < len(parts):
            raise RuntimeError("Can't concatenate edgelists with and without weight field.")
        weight = torch.cat([p.weight.expand((len(p),)) for p in parts]) if weighted else None
        scalars = {int(p.rel) if p.has_scalar_relation_type() else None for p in parts}
        if len(scalars) == 1 and None not in scalars:
            rel = torch.tensor(scalars.pop(), dtype=torch.long)
        else:
            rel = torch.cat([p.get_relation_type_as_vector() for p in parts])
        return cls(EntityList.cat([p.lhs for p in parts]), EntityList.cat([p.rhs for p in parts]), rel, weight)

    def __len__(self) -> int:
        return len(self.lhs)

    # -- relation -----------------------------------------------------------
    def has_scalar_relation_type(self) -> bool:
        return self.rel.dim() == 0

    def get_relation_type_as_scalar(self) -> int:
        if not self.has_scalar_relation_type():
            raise RuntimeError("The relation isn't a scalar")
        return int(self.rel)

    def get_relation_type_as_vector(self) -> LongTensorType:
        return self.rel.expand((len(self),)) if self.has_scalar_relation_type() else self.rel

    def get_relation_type(self) -> Union[int, LongTensorType]:
        return int(self.rel) if self.has_scalar_relation_type() else self.rel

    # -- weight -------------------------------------------------------------
    def has_weight(self) -> bool:
        return self.weight is not None

    def get_weight(self) -> Union[float, torch.Tensor]:
        return 1 if self.weight is None else self.weight

    # -- slicing, moving, comparing -------------------------------------------
    def __getitem__(self, index: Union[int, slice, LongTensorType]) -> "EdgeList":
        if _is_long(index):
            if index.dim() != 1:
                raise ValueError(f"an index tensor is 1-dimensional, got {index.dim()} dimensions")
        elif not isinstance(index, (int, slice)):
            raise TypeError(f"an EdgeList is indexed by an int, a slice or an int64 tensor, got {type(index).__name__}")
        rel = self.rel if self.has_scalar_relation_type() else self.rel[index]
        weight = None if self.weight is None else self.weight[index]
        return type(self)(self.lhs[index], self.rhs[index], rel, weight)

    def to(self, *args, **kwargs) -> "EdgeList":
        move = lambda t: t.to(*args, **kwargs)
        return type(self)(move(self.lhs), move(self.rhs), move(self.rel), None if self.weight is None else move(self.weight))

    def __eq__(self, other: Any) -> bool:
        if not isinstance(other, EdgeList):
            return NotImplemented
        return self.lhs == other.lhs and self.rhs == other.rhs and torch.equal(self.rel, other.rel)

    def __repr__(self) -> str:
        return f"EdgeList({self.lhs!r}, {self.rhs!r}, {self.rel!r}, {self.weight!r})"

    __str__ = __repr__
