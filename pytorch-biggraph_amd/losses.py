"""Loss functions (reference: torchbiggraph/losses.py): same registry
(``LOSS_FUNCTIONS``), names, constructor and ``forward(pos[P], neg[P, N],
weight[P] or None) -> 0-dim tensor`` contract; the arithmetic runs in libpbg_hip
(pbg_loss_forward / pbg_loss_backward) and is differentiable."""
from abc import ABC, abstractmethod
from typing import Optional

import torch
import torch.nn as nn

from . import _lib
from ._lib import LOSS_CODES, check
from .native import _need, _ptr, _stream
from .plugin import PluginRegistry
from .types import FloatTensorType
from .util import match_shape


class _LossFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, code, margin, pos, neg, weight):
        pos = pos.contiguous()
        neg = neg.contiguous()
        _need(pos, torch.float32, "pos_scores")
        _need(neg, torch.float32, "neg_scores")
        num_pos, num_neg = pos.shape[0], neg.shape[1]
        w = weight.contiguous().to(torch.float32) if weight is not None else None
        out = torch.empty((), dtype=torch.float32, device=pos.device)
        rows = torch.empty(max(num_pos, 1), dtype=torch.float32, device=pos.device)
        check(_lib.lib().pbg_loss_forward(code, float(margin), num_pos, num_neg, _ptr(pos), _ptr(neg), _ptr(w),
                                          _ptr(out), _ptr(rows), _stream()))
        ctx.code, ctx.margin, ctx.has_w = code, float(margin), w is not None
        ctx.save_for_backward(pos, neg, w if w is not None else pos.new_empty(0))
        return out

    @staticmethod
    def backward(ctx, upstream):
        pos, neg, w = ctx.saved_tensors
        dpos = torch.zeros_like(pos)
        dneg = torch.zeros_like(neg)
        up = upstream.contiguous().to(torch.float32)
        check(_lib.lib().pbg_loss_backward(ctx.code, ctx.margin, pos.shape[0], neg.shape[1], _ptr(pos), _ptr(neg),
                                           _ptr(w) if ctx.has_w else None, _ptr(up), _ptr(dpos), _ptr(dneg), _stream()))
        return None, None, dpos, dneg, None


class AbstractLossFunction(nn.Module, ABC):
    """Weighted loss of the scores of positive pairs (a vector of size P) and of
    negative pairs (P x N) (losses.py:20-47)."""

    loss_name: str = ""

    def __init__(self, **kwargs):
        super().__init__()

    @property
    def loss_code(self) -> int:
        return LOSS_CODES[self.loss_name]

    @property
    def fused_margin(self) -> float:
        return 0.0

    @abstractmethod
    def forward(self, pos_scores: FloatTensorType, neg_scores: FloatTensorType,
                weight: Optional[FloatTensorType]) -> FloatTensorType:
        pass

    def _run(self, pos_scores, neg_scores, weight, margin=0.0):
        num_pos = match_shape(pos_scores, -1)
        match_shape(neg_scores, num_pos, -1)
        if weight is not None:
            match_shape(weight, num_pos)
        return _LossFunction.apply(self.loss_code, margin, pos_scores, neg_scores, weight)


LOSS_FUNCTIONS = PluginRegistry[AbstractLossFunction]()


@LOSS_FUNCTIONS.register_as("logistic")
class LogisticLossFunction(AbstractLossFunction):
    loss_name = "logistic"

    def forward(self, pos_scores, neg_scores, weight):
        return self._run(pos_scores, neg_scores, weight)


@LOSS_FUNCTIONS.register_as("ranking")
class RankingLossFunction(AbstractLossFunction):
    loss_name = "ranking"

    def __init__(self, *, margin, **kwargs):
        super().__init__()
        self.margin = margin

    @property
    def fused_margin(self) -> float:
        return float(self.margin)

    def forward(self, pos_scores, neg_scores, weight):
        return self._run(pos_scores, neg_scores, weight, self.margin)


@LOSS_FUNCTIONS.register_as("softmax")
class SoftmaxLossFunction(AbstractLossFunction):
    loss_name = "softmax"

    def forward(self, pos_scores, neg_scores, weight):
        return self._run(pos_scores, neg_scores, weight)
