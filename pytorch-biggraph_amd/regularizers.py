"""Regularizers of the training step (reference: torchbiggraph/regularizers.py).

``N3Regularizer`` keeps the reference's interface (``forward`` for standard
relations, ``forward_dynamic`` for dynamic ones, on the positives as
``forward_direction_agnostic`` passes them) in plain torch operations, for code
that calls the plugin directly.  The training step does not go through it: the
model hands ``regularizer.weight`` to pbg_train_step
(``pbg_step_desc.regularization_coef``), whose kernels add the regularizer's
gradient to the loss gradient and report its value per batch.
"""
from abc import ABC, abstractmethod
from typing import Optional

import torch

from .plugin import PluginRegistry
from .types import FloatTensorType, LongTensorType


class AbstractRegularizer(ABC):
    """A weighted penalty on the embeddings that took part in a batch's scores
    (regularizers.py:20-47)."""

    def __init__(self, weight: float):
        self.weight = weight

    @abstractmethod
    def forward_dynamic(self, src_pos: FloatTensorType, dst_pos: FloatTensorType, operator,
                        rel_idxs: LongTensorType) -> FloatTensorType:
        pass

    @abstractmethod
    def forward(self, src_pos: FloatTensorType, dst_pos: FloatTensorType, operator) -> FloatTensorType:
        pass


REGULARIZERS = PluginRegistry[AbstractRegularizer]()


@REGULARIZERS.register_as("N3")
class N3Regularizer(AbstractRegularizer):
    """Sum of cubed moduli (regularizers.py:51-97): of the positives' embeddings
    as the operator presents them (`prepare_embs_for_reg`) and of the operator's
    parameters (`get_operator_params_for_reg`), the latter once per edge for
    dynamic relations and once per element of `src_pos`'s leading axis otherwise."""

    def forward_dynamic(self, src_pos, dst_pos, operator, rel_idxs):
        total = 0
        operator_params = operator.get_operator_params_for_reg(rel_idxs)
        if operator_params is not None:
            total = total + torch.sum(operator_params.to(src_pos.device) ** 3)
        for x in (src_pos, dst_pos):
            total = total + torch.sum(operator.prepare_embs_for_reg(x) ** 3)
        return total * self.weight

    def forward(self, src_pos, dst_pos, operator):
        total = 0
        operator_params = operator.get_operator_params_for_reg()
        if operator_params is not None:
            total = total + torch.sum(operator_params.to(src_pos.device) ** 3) * len(src_pos)
        for x in (src_pos, dst_pos):
            total = total + torch.sum(operator.prepare_embs_for_reg(x) ** 3)
        return total * self.weight
