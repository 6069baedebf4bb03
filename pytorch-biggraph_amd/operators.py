"""Relation operators (reference: torchbiggraph/operators.py).

Same registries (``OPERATORS`` / ``DYNAMIC_OPERATORS``), class names,
constructor signatures, parameter names, shapes and initial values as the
reference; ``forward`` runs in libpbg_hip (pbg_operator_forward / _backward)
and is differentiable.  Each class also carries the operator code the fused
training step uses.
"""
from abc import ABC, abstractmethod
from typing import Optional, Union

import torch
import torch.nn as nn

from . import _lib
from ._lib import OPERATOR_CODES, check
from .native import _need, _ptr, _stream
from .plugin import PluginRegistry
from .types import FloatTensorType, LongTensorType, Side
from .util import match_shape


class _OperatorFunction(torch.autograd.Function):
    """y = op(x); gradients for x and the operator parameters."""

    @staticmethod
    def forward(ctx, code, embeddings, p0, p1, rel):
        x = embeddings.contiguous()
        _need(x, torch.float32, "embeddings")
        dim = x.shape[-1]
        rows = x.numel() // dim if dim > 0 else 0
        y = torch.empty_like(x)
        num_ops = 1
        relc = None
        if rel is not None:
            relc = rel.contiguous().to(device=x.device)
            _need(relc, torch.int64, "operator_idxs")
            num_ops = p0.shape[0] if p0 is not None else 1
        p0c = p0.contiguous() if p0 is not None else None
        p1c = p1.contiguous() if p1 is not None else None
        check(_lib.lib().pbg_operator_forward(code, dim, rows, _ptr(x), _ptr(p0c), _ptr(p1c), _ptr(relc), num_ops,
                                              _ptr(y), _stream()))
        ctx.code, ctx.dim, ctx.rows, ctx.num_ops = code, dim, rows, num_ops
        ctx.save_for_backward(x, p0c if p0c is not None else x.new_empty(0), p1c if p1c is not None else x.new_empty(0),
                              relc if relc is not None else torch.empty(0, dtype=torch.int64, device=x.device))
        ctx.has = (p0 is not None, p1 is not None, rel is not None)
        return y

    @staticmethod
    def backward(ctx, dy):
        x, p0, p1, rel = ctx.saved_tensors
        has_p0, has_p1, has_rel = ctx.has
        dy = dy.contiguous()
        dx = torch.empty_like(x)
        dp0 = torch.zeros_like(p0) if has_p0 else None
        dp1 = torch.zeros_like(p1) if has_p1 else None
        check(_lib.lib().pbg_operator_backward(
            ctx.code, ctx.dim, ctx.rows, _ptr(x), _ptr(dy), _ptr(p0) if has_p0 else None, _ptr(p1) if has_p1 else None,
            _ptr(rel) if has_rel else None, ctx.num_ops, _ptr(dx), _ptr(dp0), _ptr(dp1), _stream()))
        return None, dx, dp0, dp1, None


class AbstractOperator(nn.Module, ABC):
    """The same operation, with one set of parameters, on many vectors (the last
    axis of the input); output has the input's shape (operators.py:19-43)."""

    op_name: str = "none"

    def __init__(self, dim: int):
        super().__init__()
        self.dim = dim

    @property
    def op_code(self) -> int:
        return OPERATOR_CODES[self.op_name]

    def fused_params(self):
        """(p0, p1) in the layout of pbg_step_buffers."""
        return None, None

    @abstractmethod
    def forward(self, embeddings: FloatTensorType) -> FloatTensorType:
        pass

    def get_operator_params_for_reg(self) -> Optional[FloatTensorType]:
        raise NotImplementedError("Regularizer not implemented for this operator")

    def prepare_embs_for_reg(self, embs: FloatTensorType) -> FloatTensorType:
        return embs.abs()

    def _run(self, embeddings: FloatTensorType) -> FloatTensorType:
        match_shape(embeddings, ..., self.dim)
        p0, p1 = self.fused_params()
        return _OperatorFunction.apply(self.op_code, embeddings, p0, p1, None)


OPERATORS = PluginRegistry[AbstractOperator]()


@OPERATORS.register_as("none")
class IdentityOperator(AbstractOperator):
    op_name = "none"

    def forward(self, embeddings: FloatTensorType) -> FloatTensorType:
        match_shape(embeddings, ..., self.dim)
        return embeddings

    def get_operator_params_for_reg(self) -> Optional[FloatTensorType]:
        return None


@OPERATORS.register_as("diagonal")
class DiagonalOperator(AbstractOperator):
    op_name = "diagonal"

    def __init__(self, dim: int):
        super().__init__(dim)
        self.diagonal = nn.Parameter(torch.ones((self.dim,)))

    def fused_params(self):
        return self.diagonal, None

    def forward(self, embeddings: FloatTensorType) -> FloatTensorType:
        return self._run(embeddings)

    def get_operator_params_for_reg(self) -> Optional[FloatTensorType]:
        return self.diagonal.abs()


@OPERATORS.register_as("translation")
class TranslationOperator(AbstractOperator):
    op_name = "translation"

    def __init__(self, dim: int):
        super().__init__(dim)
        self.translation = nn.Parameter(torch.zeros((self.dim,)))

    def fused_params(self):
        return self.translation, None

    def forward(self, embeddings: FloatTensorType) -> FloatTensorType:
        return self._run(embeddings)

    def get_operator_params_for_reg(self) -> Optional[FloatTensorType]:
        return self.translation.abs()


@OPERATORS.register_as("linear")
class LinearOperator(AbstractOperator):
    op_name = "linear"

    def __init__(self, dim: int):
        super().__init__(dim)
        self.linear_transformation = nn.Parameter(torch.eye(self.dim))

    def fused_params(self):
        return self.linear_transformation, None

    def forward(self, embeddings: FloatTensorType) -> FloatTensorType:
        return self._run(embeddings)


@OPERATORS.register_as("affine")
class AffineOperator(AbstractOperator):
    """y = A x + t (operators.py:102-115)."""

    op_name = "affine"

    def __init__(self, dim: int):
        super().__init__(dim)
        self.linear_transformation = nn.Parameter(torch.eye(self.dim))
        self.translation = nn.Parameter(torch.zeros((self.dim,)))

    def fused_params(self):
        return self.linear_transformation, self.translation

    def forward(self, embeddings: FloatTensorType) -> FloatTensorType:
        return self._run(embeddings)


@OPERATORS.register_as("complex_diagonal")
class ComplexDiagonalOperator(AbstractOperator):
    op_name = "complex_diagonal"

    def __init__(self, dim: int):
        super().__init__(dim)
        if dim % 2 != 0:
            raise ValueError("Need even dimension as 1st half is real and 2nd half is imaginary coordinates")
        self.real = nn.Parameter(torch.ones((self.dim // 2,)))
        self.imag = nn.Parameter(torch.zeros((self.dim // 2,)))

    def fused_params(self):
        return self.real, self.imag

    def forward(self, embeddings: FloatTensorType) -> FloatTensorType:
        return self._run(embeddings)

    def get_operator_params_for_reg(self) -> Optional[FloatTensorType]:
        return torch.sqrt(self.real ** 2 + self.imag ** 2)

    def prepare_embs_for_reg(self, embs: FloatTensorType) -> FloatTensorType:
        assert embs.shape[-1] == self.dim
        real, imag = embs[..., : self.dim // 2], embs[..., self.dim // 2:]
        return torch.sqrt(real ** 2 + imag ** 2)


class AbstractDynamicOperator(nn.Module, ABC):
    """Different operations of one kind, each with its own parameters, selected
    per vector by an index tensor shaped like the input without its last axis
    (operators.py:160-191)."""

    op_name: str = "none"

    def __init__(self, dim: int, num_operations: int):
        super().__init__()
        self.dim = dim
        self.num_operations = num_operations

    @property
    def op_code(self) -> int:
        return OPERATOR_CODES[self.op_name]

    def fused_params(self):
        return None, None

    @abstractmethod
    def forward(self, embeddings: FloatTensorType, operator_idxs: LongTensorType) -> FloatTensorType:
        pass

    def get_operator_params_for_reg(self, operator_idxs: LongTensorType) -> Optional[FloatTensorType]:
        raise NotImplementedError("Regularizer not implemented for this operator")

    def prepare_embs_for_reg(self, embs: FloatTensorType) -> FloatTensorType:
        return embs.abs()

    def _run(self, embeddings: FloatTensorType, operator_idxs: LongTensorType) -> FloatTensorType:
        match_shape(embeddings, ..., self.dim)
        match_shape(operator_idxs, *embeddings.size()[:-1])
        p0, p1 = self.fused_params()
        return _OperatorFunction.apply(self.op_code, embeddings, p0, p1, operator_idxs)


DYNAMIC_OPERATORS = PluginRegistry[AbstractDynamicOperator]()


@DYNAMIC_OPERATORS.register_as("none")
class IdentityDynamicOperator(AbstractDynamicOperator):
    op_name = "none"

    def forward(self, embeddings: FloatTensorType, operator_idxs: LongTensorType) -> FloatTensorType:
        match_shape(embeddings, ..., self.dim)
        match_shape(operator_idxs, *embeddings.size()[:-1])
        return embeddings

    def get_operator_params_for_reg(self, operator_idxs: LongTensorType) -> Optional[FloatTensorType]:
        return None


@DYNAMIC_OPERATORS.register_as("diagonal")
class DiagonalDynamicOperator(AbstractDynamicOperator):
    op_name = "diagonal"

    def __init__(self, dim: int, num_operations: int):
        super().__init__(dim, num_operations)
        self.diagonals = nn.Parameter(torch.ones((self.num_operations, self.dim)))

    def fused_params(self):
        return self.diagonals, None

    def forward(self, embeddings: FloatTensorType, operator_idxs: LongTensorType) -> FloatTensorType:
        return self._run(embeddings, operator_idxs)

    def get_operator_params_for_reg(self, operator_idxs: LongTensorType) -> Optional[FloatTensorType]:
        return self.diagonals.to(device=operator_idxs.device)[operator_idxs].abs()


@DYNAMIC_OPERATORS.register_as("translation")
class TranslationDynamicOperator(AbstractDynamicOperator):
    op_name = "translation"

    def __init__(self, dim: int, num_operations: int):
        super().__init__(dim, num_operations)
        self.translations = nn.Parameter(torch.zeros((self.num_operations, self.dim)))

    def fused_params(self):
        return self.translations, None

    def forward(self, embeddings: FloatTensorType, operator_idxs: LongTensorType) -> FloatTensorType:
        return self._run(embeddings, operator_idxs)

    def get_operator_params_for_reg(self, operator_idxs: LongTensorType) -> Optional[FloatTensorType]:
        return self.translations.to(device=operator_idxs.device)[operator_idxs].abs()


@DYNAMIC_OPERATORS.register_as("linear")
class LinearDynamicOperator(AbstractDynamicOperator):
    op_name = "linear"

    def __init__(self, dim: int, num_operations: int):
        super().__init__(dim, num_operations)
        self.linear_transformations = nn.Parameter(torch.diag_embed(torch.ones(()).expand(num_operations, dim)))

    def fused_params(self):
        return self.linear_transformations, None

    def forward(self, embeddings: FloatTensorType, operator_idxs: LongTensorType) -> FloatTensorType:
        return self._run(embeddings, operator_idxs)


@DYNAMIC_OPERATORS.register_as("affine")
class AffineDynamicOperator(AbstractDynamicOperator):
    """y_i = A[idx_i] x_i + t[idx_i] (operators.py:272-293)."""

    op_name = "affine"

    def __init__(self, dim: int, num_operations: int):
        super().__init__(dim, num_operations)
        self.linear_transformations = nn.Parameter(torch.diag_embed(torch.ones(()).expand(num_operations, dim)))
        self.translations = nn.Parameter(torch.zeros((self.num_operations, self.dim)))

    def fused_params(self):
        return self.linear_transformations, self.translations

    def forward(self, embeddings: FloatTensorType, operator_idxs: LongTensorType) -> FloatTensorType:
        return self._run(embeddings, operator_idxs)


@DYNAMIC_OPERATORS.register_as("complex_diagonal")
class ComplexDiagonalDynamicOperator(AbstractDynamicOperator):
    op_name = "complex_diagonal"

    def __init__(self, dim: int, num_operations: int):
        super().__init__(dim, num_operations)
        if dim % 2 != 0:
            raise ValueError("Need even dimension as 1st half is real and 2nd half is imaginary coordinates")
        self.real = nn.Parameter(torch.ones((self.num_operations, self.dim // 2)))
        self.imag = nn.Parameter(torch.zeros((self.num_operations, self.dim // 2)))

    def fused_params(self):
        return self.real, self.imag

    def forward(self, embeddings: FloatTensorType, operator_idxs: LongTensorType) -> FloatTensorType:
        return self._run(embeddings, operator_idxs)

    def get_operator_params_for_reg(self, operator_idxs) -> Optional[FloatTensorType]:
        return torch.sqrt(self.real[operator_idxs] ** 2 + self.imag[operator_idxs] ** 2)

    def prepare_embs_for_reg(self, embs: FloatTensorType) -> FloatTensorType:
        assert embs.shape[-1] == self.dim
        real, imag = embs[..., : self.dim // 2], embs[..., self.dim // 2:]
        return torch.sqrt(real ** 2 + imag ** 2)


def instantiate_operator(
    operator: str, side: Side, num_dynamic_rels: int, dim: int
) -> Optional[Union[AbstractOperator, AbstractDynamicOperator]]:
    """operators.py:341-351: dynamic relations get one dynamic operator per side;
    otherwise only the right-hand side has an operator."""
    if num_dynamic_rels > 0:
        return DYNAMIC_OPERATORS.get_class(operator)(dim, num_dynamic_rels)
    if side is Side.LHS:
        return None
    return OPERATORS.get_class(operator)(dim)
