"""Small shared types (reference: torchbiggraph/types.py:23-68)."""
from enum import Enum
from typing import NamedTuple, TypeVar

import torch

FloatTensorType = torch.Tensor  # float32
LongTensorType = torch.Tensor  # int64
T = TypeVar("T")


class Side(Enum):
    LHS = 0
    RHS = 1

    def pick(self, lhs: T, rhs: T) -> T:
        if self is Side.LHS:
            return lhs
        if self is Side.RHS:
            return rhs
        raise NotImplementedError("Unknown side: %s" % self)


EntityName = str
Partition = int


class Bucket(NamedTuple):
    lhs: Partition
    rhs: Partition

    def get_partition(self, side: Side) -> Partition:
        return side.pick(self.lhs, self.rhs)

    def __str__(self) -> str:
        return "( %d , %d )" % (self.lhs, self.rhs)


UNPARTITIONED: Partition = 0
