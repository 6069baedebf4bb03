"""Type aliases and the two small value types of the step's interface
(reference: torchbiggraph/types.py:23-68): ``Side`` and ``Bucket``."""
import enum
import typing

import torch

T = typing.TypeVar("T")

# Annotations only: every tensor is a torch.Tensor, the alias states the dtype.
LongTensorType = torch.Tensor   # int64 indices
FloatTensorType = torch.Tensor  # float32 values

Partition = int
EntityName = str
UNPARTITIONED: Partition = 0  # the partition number of an entity type that is not partitioned


class Side(enum.Enum):
    """Left- or right-hand side of an edge."""

    LHS = 0
    RHS = 1

    def pick(self, lhs: T, rhs: T) -> T:
        """`lhs` for Side.LHS, `rhs` for Side.RHS."""
        return (lhs, rhs)[self.value]


class Bucket(typing.NamedTuple):
    """The edges whose left entities lie in partition `lhs` and whose right
    entities lie in partition `rhs`."""

    lhs: Partition
    rhs: Partition

    def __str__(self) -> str:
        return f"( {self.lhs:d} , {self.rhs:d} )"

    def get_partition(self, side: Side) -> Partition:
        return self[side.value]
