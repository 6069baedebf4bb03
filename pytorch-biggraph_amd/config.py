"""The few schema fields that parameterise the step (reference:
torchbiggraph/config.py:54-133 EntitySchema / RelationSchema).  The full config
system of the reference is out of scope; these are plain records with the same
attribute names."""
from dataclasses import dataclass
from typing import Optional


@dataclass
class EntitySchema:
    num_partitions: int = 1
    featurized: bool = False
    dimension: Optional[int] = None


@dataclass
class RelationSchema:
    name: str
    lhs: str
    rhs: str
    weight: float = 1.0
    operator: str = "none"
    all_negs: bool = False
