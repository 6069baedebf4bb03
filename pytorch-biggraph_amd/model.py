"""Embeddings, comparators and the multi-relation model (reference:
torchbiggraph/model.py).

``COMPARATORS`` holds ``dot``, ``cos``, ``l2`` and ``squared_l2`` with the reference's
``prepare`` / ``forward`` contract (differentiable, computed by
pbg_comparator_*).  ``MultiRelationEmbedder`` keeps the reference's constructor,
``set_embeddings`` / ``set_all_embeddings`` / ``clear_all_embeddings`` and
``forward(edges) -> (Scores, reg)``; its forward is ONE call into libpbg_hip
(pbg_model_forward) and additionally accepts the uniform-negative indices from
outside, so that two implementations can be fed the same negatives.  Training
goes through ``train.Trainer`` (one pbg_train_step call per batch), not through
autograd on these scores.

``regularizer``: an ``N3Regularizer`` (the one the reference registers); the
training step takes its weight, ``forward`` returns its value as the reference's
does.

``half_precision`` (model.py:504-505: embeddings become float16 once prepared for the
comparator; "GPU ONLY", config.py:496-498) is taken for the dot and cos comparators
without bias and regularizer; the step refuses the other combinations.

Not provided (outside the accelerated path): FeaturizedEmbedding.
"""
from abc import ABC, abstractmethod
from enum import Enum
from typing import Dict, List, NamedTuple, Optional, Sequence, Tuple, Union

import torch
import torch.nn as nn

from . import _lib, native
from ._lib import COMPARATOR_CODES, check
from .config import EntitySchema, RelationSchema
from .edgelist import EdgeList
from .entitylist import EntityList
from .native import _need, _ptr, _stream
from .regularizers import AbstractRegularizer, N3Regularizer
from .operators import AbstractDynamicOperator, AbstractOperator
from .plugin import PluginRegistry
from .types import Bucket, FloatTensorType, LongTensorType, Side
from .util import match_shape


class AbstractEmbedding(nn.Module, ABC):
    @abstractmethod
    def forward(self, input_: EntityList) -> FloatTensorType:
        pass

    @abstractmethod
    def get_all_entities(self) -> FloatTensorType:
        pass

    @abstractmethod
    def sample_entities(self, *dims: int) -> FloatTensorType:
        pass


class _GatherFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, weight, idx):
        ctx.save_for_backward(idx)
        ctx.shape = weight.shape
        return native.gather_rows(weight.detach().contiguous(), idx.contiguous())

    @staticmethod
    def backward(ctx, grad):
        (idx,) = ctx.saved_tensors
        # a sparse COO gradient, as F.embedding(sparse=True) produces
        flat = idx.reshape(1, -1)
        sparse = torch.sparse_coo_tensor(flat, grad.reshape(-1, ctx.shape[1]), ctx.shape)
        return sparse, None


class SimpleEmbedding(AbstractEmbedding):
    """Row gather from one table (model.py:51-75)."""

    def __init__(self, weight: nn.Parameter, max_norm: Optional[float] = None):
        super().__init__()
        self.weight: nn.Parameter = weight
        self.max_norm: Optional[float] = max_norm

    def forward(self, input_: EntityList) -> FloatTensorType:
        return self.get(input_.to_tensor())

    def get(self, input_: LongTensorType) -> FloatTensorType:
        if input_.numel() == 0:
            return self.weight.new_empty((*input_.shape, self.weight.shape[1]))
        if self.max_norm is not None:  # F.embedding(max_norm=...): the table itself is renormalised first
            native.embedding_renorm_(self.weight.data, input_, self.max_norm)
        return _GatherFunction.apply(self.weight, input_)

    def get_all_entities(self) -> FloatTensorType:
        return self.get(torch.arange(self.weight.size(0), dtype=torch.long, device=self.weight.device))

    def sample_indices(self, *dims: int) -> LongTensorType:
        return torch.randint(low=0, high=self.weight.size(0), size=dims, device=self.weight.device)

    def sample_entities(self, *dims: int) -> FloatTensorType:
        return self.get(self.sample_indices(*dims))


# ---------------------------------------------------------------------------
class _PrepareFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, code, embs):
        x = embs.contiguous()
        _need(x, torch.float32, "embs")
        dim = x.shape[-1]
        n = x.numel() // dim if dim else 0
        y = torch.empty_like(x)
        aux = torch.empty(max(n, 1), dtype=torch.float32, device=x.device)
        check(_lib.lib().pbg_comparator_prepare(code, dim, n, _ptr(x), _ptr(y), _ptr(aux), _stream()))
        ctx.code, ctx.dim, ctx.n = code, dim, n
        ctx.save_for_backward(y, aux)
        return y

    @staticmethod
    def backward(ctx, dy):
        y, aux = ctx.saved_tensors
        dy = dy.contiguous()
        dx = torch.empty_like(y)
        check(_lib.lib().pbg_comparator_prepare_backward(ctx.code, ctx.dim, ctx.n, _ptr(dy), _ptr(y), _ptr(aux),
                                                         _ptr(dx), _stream()))
        return None, dx


class _ScoresFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, code, lhs_pos, rhs_pos, lhs_neg, rhs_neg):
        ts = [t.contiguous() for t in (lhs_pos, rhs_pos, lhs_neg, rhs_neg)]
        for t, name in zip(ts, ("lhs_pos", "rhs_pos", "lhs_neg", "rhs_neg")):
            _need(t, torch.float32, name)
        c, p, d = ts[0].shape
        ln, rn = ts[2].shape[1], ts[3].shape[1]
        dev = ts[0].device
        pos = torch.empty((c, p), dtype=torch.float32, device=dev)
        lneg = torch.empty((c, p, ln), dtype=torch.float32, device=dev)
        rneg = torch.empty((c, p, rn), dtype=torch.float32, device=dev)
        nbytes = _lib.lib().pbg_comparator_workspace_bytes(c, p, ln, rn)
        ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=dev)
        check(_lib.lib().pbg_comparator_forward(code, c, p, ln, rn, d, *[_ptr(t) for t in ts], _ptr(pos), _ptr(lneg),
                                                _ptr(rneg), _ptr(ws), ws.numel(), _stream()))
        ctx.code, ctx.dims = code, (c, p, ln, rn, d)
        ctx.save_for_backward(*ts, pos, lneg, rneg)
        return pos, lneg, rneg

    @staticmethod
    def backward(ctx, dpos, dlneg, drneg):
        lp, rp, ln_, rn_, pos, lneg, rneg = ctx.saved_tensors
        c, p, ln, rn, d = ctx.dims
        dev = lp.device
        grads = [g.contiguous() if g is not None else torch.zeros_like(ref)
                 for g, ref in ((dpos, pos), (dlneg, lneg), (drneg, rneg))]
        outs = [torch.empty_like(t) for t in (lp, rp, ln_, rn_)]
        nbytes = _lib.lib().pbg_comparator_workspace_bytes(c, p, ln, rn)
        ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=dev)
        check(_lib.lib().pbg_comparator_backward(
            ctx.code, c, p, ln, rn, d, _ptr(lp), _ptr(rp), _ptr(ln_), _ptr(rn_), _ptr(pos), _ptr(lneg), _ptr(rneg),
            *[_ptr(g) for g in grads], *[_ptr(o) for o in outs], _ptr(ws), ws.numel(), _stream()))
        return (None, *outs)


class AbstractComparator(nn.Module, ABC):
    """Scores between sets of vectors chunked alike:
    L+ [C,P,D], R+ [C,P,D], L- [C,L,D], R- [C,R,D] ->
    <L+,R+> [C,P], R+ x L- [C,P,L], L+ x R- [C,P,R]   (model.py:105-153)."""

    comparator_name: str = ""

    @property
    def comparator_code(self) -> int:
        return COMPARATOR_CODES[self.comparator_name]

    def prepare(self, embs: FloatTensorType) -> FloatTensorType:
        return embs

    def forward(self, lhs_pos, rhs_pos, lhs_neg, rhs_neg) -> Tuple[FloatTensorType, FloatTensorType, FloatTensorType]:
        num_chunks, num_pos_per_chunk, dim = match_shape(lhs_pos, -1, -1, -1)
        match_shape(rhs_pos, num_chunks, num_pos_per_chunk, dim)
        match_shape(lhs_neg, num_chunks, -1, dim)
        match_shape(rhs_neg, num_chunks, -1, dim)
        return _ScoresFunction.apply(self.comparator_code, lhs_pos, rhs_pos, lhs_neg, rhs_neg)


COMPARATORS = PluginRegistry[AbstractComparator]()


@COMPARATORS.register_as("dot")
class DotComparator(AbstractComparator):
    comparator_name = "dot"


@COMPARATORS.register_as("cos")
class CosComparator(AbstractComparator):
    comparator_name = "cos"

    def prepare(self, embs: FloatTensorType) -> FloatTensorType:
        return _PrepareFunction.apply(self.comparator_code, embs)


@COMPARATORS.register_as("l2")
class L2Comparator(AbstractComparator):
    comparator_name = "l2"


@COMPARATORS.register_as("squared_l2")
class SquaredL2Comparator(AbstractComparator):
    """Negative squared distance (model.py:281-305)."""

    comparator_name = "squared_l2"


class BiasedComparator(AbstractComparator):
    """config.bias (model.py:306-344,902-903): the first coordinate of every
    embedding is a bias -- it stays out of the wrapped comparator and is added
    to the scores of its row.  Inside the training step the same thing is the
    ``bias`` field of the step description."""

    def __init__(self, base_comparator: AbstractComparator):
        super().__init__()
        self.base_comparator = base_comparator

    @property
    def comparator_name(self) -> str:
        return self.base_comparator.comparator_name

    def prepare(self, embs: FloatTensorType) -> FloatTensorType:
        return torch.cat([embs[..., :1], self.base_comparator.prepare(embs[..., 1:])], dim=-1)

    def forward(self, lhs_pos, rhs_pos, lhs_neg, rhs_neg) -> Tuple[FloatTensorType, FloatTensorType, FloatTensorType]:
        num_chunks, num_pos_per_chunk, dim = match_shape(lhs_pos, -1, -1, -1)
        match_shape(rhs_pos, num_chunks, num_pos_per_chunk, dim)
        match_shape(lhs_neg, num_chunks, -1, dim)
        match_shape(rhs_neg, num_chunks, -1, dim)
        pos_scores, lhs_neg_scores, rhs_neg_scores = self.base_comparator(
            lhs_pos[..., 1:], rhs_pos[..., 1:], lhs_neg[..., 1:], rhs_neg[..., 1:])
        lhs_pos_bias = lhs_pos[..., 0]
        rhs_pos_bias = rhs_pos[..., 0]
        pos_scores = pos_scores + lhs_pos_bias + rhs_pos_bias
        lhs_neg_scores = lhs_neg_scores + rhs_pos_bias.unsqueeze(-1) + lhs_neg[..., 0].unsqueeze(-2)
        rhs_neg_scores = rhs_neg_scores + lhs_pos_bias.unsqueeze(-1) + rhs_neg[..., 0].unsqueeze(-2)
        return pos_scores, lhs_neg_scores, rhs_neg_scores


# ---------------------------------------------------------------------------
def ceil_of_ratio(num: int, den: int) -> int:
    return (num - 1) // den + 1


class Negatives(Enum):
    NONE = "none"
    UNIFORM = "uniform"
    BATCH_UNIFORM = "batch_uniform"
    ALL = "all"


class Scores(NamedTuple):
    lhs_pos: FloatTensorType
    rhs_pos: FloatTensorType
    lhs_neg: FloatTensorType
    rhs_neg: FloatTensorType


class RankOutput(NamedTuple):
    """forward_ranks: per edge, without the [B, N] score matrices."""
    lhs_pos: FloatTensorType
    rhs_pos: FloatTensorType
    ranks: Tuple[torch.Tensor, torch.Tensor]  # (lhs, rhs): 1 + negatives scoring at least as high as the positive
    loss_edge: FloatTensorType                # relation weight x edge weight x (lhs loss + rhs loss)
    auc_hits: Optional[torch.Tensor]          # [2]: random (positive, negative) pairs with positive > negative
    has_negs: Tuple[bool, bool]               # a side without negatives has no rank


class MultiRelationEmbedder(nn.Module):
    """A multi-relation embedding model scored against batch and uniform
    negatives (model.py:368-856)."""

    EMB_PREFIX = "emb_"

    def __init__(
        self,
        default_dim: int,
        relations: List[RelationSchema],
        entities: Dict[str, EntitySchema],
        num_batch_negs: int,
        num_uniform_negs: int,
        disable_lhs_negs: bool,
        disable_rhs_negs: bool,
        lhs_operators: Sequence[Optional[Union[AbstractOperator, AbstractDynamicOperator]]],
        rhs_operators: Sequence[Optional[Union[AbstractOperator, AbstractDynamicOperator]]],
        comparator: AbstractComparator,
        regularizer=None,
        global_emb: bool = False,
        max_norm: Optional[float] = None,
        num_dynamic_rels: int = 0,
        half_precision: bool = False,
    ) -> None:
        super().__init__()
        if regularizer is not None and not isinstance(regularizer, N3Regularizer):
            raise NotImplementedError("Only the N3 regularizer is supported")
        if any(e.featurized for e in entities.values()):
            raise NotImplementedError("Featurized entities are not supported")
        self.default_dim = default_dim
        self.relations: List[RelationSchema] = relations
        self.entities: Dict[str, EntitySchema] = entities
        self.num_dynamic_rels: int = num_dynamic_rels
        if num_dynamic_rels > 0:
            assert len(relations) == 1
        self.lhs_operators: nn.ModuleList = nn.ModuleList(lhs_operators)
        self.rhs_operators: nn.ModuleList = nn.ModuleList(rhs_operators)
        self.num_batch_negs: int = num_batch_negs
        self.num_uniform_negs: int = num_uniform_negs
        self.disable_lhs_negs = disable_lhs_negs
        self.disable_rhs_negs = disable_rhs_negs
        self.comparator = comparator
        self.lhs_embs: nn.ModuleDict = nn.ModuleDict()
        self.rhs_embs: nn.ModuleDict = nn.ModuleDict()
        # model.py:433-441: one learned vector per entity type, zeros at first
        self.global_embs: Optional[nn.ParameterDict] = None
        if global_emb:
            self.global_embs = nn.ParameterDict({
                self.EMB_PREFIX + entity: nn.Parameter(torch.zeros((schema.dimension or default_dim,)))
                for entity, schema in entities.items()})
        self.max_norm: Optional[float] = max_norm
        self.half_precision = bool(half_precision)
        self.regularizer: Optional[AbstractRegularizer] = regularizer
        self._runners: Dict[tuple, native.StepRunner] = {}

    # --- embeddings ---------------------------------------------------------
    def set_embeddings(self, entity: str, side: Side, weights: nn.Parameter) -> None:
        emb = SimpleEmbedding(weights, max_norm=self.max_norm)
        side.pick(self.lhs_embs, self.rhs_embs)[self.EMB_PREFIX + entity] = emb
        self._runners.clear()

    def set_all_embeddings(self, holder, bucket: Bucket) -> None:
        for entity in holder.lhs_unpartitioned_types:
            self.set_embeddings(entity, Side.LHS, holder.unpartitioned_embeddings[entity])
        for entity in holder.rhs_unpartitioned_types:
            self.set_embeddings(entity, Side.RHS, holder.unpartitioned_embeddings[entity])
        for entity in holder.lhs_partitioned_types:
            self.set_embeddings(entity, Side.LHS, holder.partitioned_embeddings[entity, bucket.lhs])
        for entity in holder.rhs_partitioned_types:
            self.set_embeddings(entity, Side.RHS, holder.partitioned_embeddings[entity, bucket.rhs])

    def clear_all_embeddings(self) -> None:
        self.lhs_embs.clear()
        self.rhs_embs.clear()
        self._runners.clear()

    # --- the fused path -------------------------------------------------------
    def resolve(self, edges: EdgeList):
        """Validates the batch as model.py:633-646,674-678 does and returns
        (relation_idx, lhs table module, rhs table module)."""
        if self.num_dynamic_rels > 0:
            if edges.has_scalar_relation_type():
                raise TypeError("Need relation for each positive pair")
            relation_idx = 0
        else:
            if not edges.has_scalar_relation_type():
                raise TypeError("All positive pairs must come from the same relation")
            relation_idx = edges.get_relation_type_as_scalar()
            if self.lhs_operators[relation_idx] is not None:
                raise RuntimeError(
                    "In non-dynamic relation mode there should be only a right-hand side operator"
                )
        relation = self.relations[relation_idx]
        lhs_module = self.lhs_embs[self.EMB_PREFIX + relation.lhs]
        rhs_module = self.rhs_embs[self.EMB_PREFIX + relation.rhs]
        return relation_idx, lhs_module, rhs_module

    def global_vectors(self, relation_idx: int):
        """(lhs, rhs) global embedding Parameters of the relation's entity types,
        or None when global embeddings are off (model.py:486-492)."""
        if self.global_embs is None:
            return None
        if self.num_dynamic_rels > 0:
            raise RuntimeError("Cannot have global embs with dynamic rels")
        relation = self.relations[relation_idx]
        return (self.global_embs[self.EMB_PREFIX + relation.lhs], self.global_embs[self.EMB_PREFIX + relation.rhs])

    def step_spec(self, relation_idx: int, num_pos: int, dim: int, **training) -> native.StepSpec:
        rhs_op = self.rhs_operators[relation_idx]
        dynamic = self.num_dynamic_rels > 0
        return native.StepSpec(
            dim=dim, batch_size=num_pos, num_workers=1, num_batch_negs=self.num_batch_negs,
            num_uniform_negs=self.num_uniform_negs, disable_lhs_negs=bool(self.disable_lhs_negs),
            disable_rhs_negs=bool(self.disable_rhs_negs),
            operator=rhs_op.op_name if rhs_op is not None else "none", dynamic=dynamic,
            num_relations=self.num_dynamic_rels if dynamic else 1,
            comparator=self.comparator.comparator_name,
            regularization_coef=float(self.regularizer.weight) if self.regularizer is not None else 0.0,
            max_norm=self.max_norm, bias=isinstance(self.comparator, BiasedComparator),
            all_negs=bool(self.relations[relation_idx].all_negs), half_precision=self.half_precision, **training)

    def operator_tensors(self, relation_idx: int):
        """({name: tensor} of the rhs operator, of the lhs operator) in the
        layout pbg_step_buffers expects."""
        def pack(op):
            if op is None:
                return {}
            p0, p1 = op.fused_params()
            if p0 is None:
                return {}
            return {"p0": p0.data, "p1": p1.data} if p1 is not None else {"p0": p0.data}
        lhs = pack(self.lhs_operators[relation_idx]) if self.num_dynamic_rels > 0 else {}
        return pack(self.rhs_operators[relation_idx]), lhs

    def sample_uniform(self, lhs_module, rhs_module, num_chunks: int):
        """torch.randint(0, E, (C, U)) per side, left-hand side first, as
        SimpleEmbedding.sample_entities draws them (model.py:70-75,802-821)."""
        u = self.num_uniform_negs
        ul = lhs_module.sample_indices(num_chunks, u) if (u > 0 and not self.disable_lhs_negs) else None
        ur = rhs_module.sample_indices(num_chunks, u) if (u > 0 and not self.disable_rhs_negs) else None
        return ul, ur

    def _regularizer_value(self, relation_idx: int, lhs_module, rhs_module, lhs, rhs, rel, chunk_size: int):
        """What forward_direction_agnostic hands the regularizer (model.py:784-801,
        845-854), per direction: the positives after operator and
        comparator.prepare, zero-padded to whole chunks, as [C, P, D]."""
        def chunked(embs, operator):
            if operator is not None:
                embs = operator(embs, rel) if self.num_dynamic_rels > 0 else operator(embs)
            embs = self.comparator.prepare(embs)
            pad = -embs.shape[0] % chunk_size
            if pad:
                embs = torch.cat((embs, embs.new_zeros((pad, embs.shape[1]))), dim=0)
            return embs.view(-1, chunk_size, embs.shape[1])

        with torch.no_grad():
            lhs_pos, rhs_pos = lhs_module.get(lhs), rhs_module.get(rhs)
            if self.num_dynamic_rels == 0:
                op = self.rhs_operators[relation_idx]
                return self.regularizer.forward(chunked(lhs_pos, None), chunked(rhs_pos, op), op)
            rhs_op, lhs_op = self.rhs_operators[relation_idx], self.lhs_operators[relation_idx]
            return (self.regularizer.forward_dynamic(chunked(lhs_pos, None), chunked(rhs_pos, rhs_op), rhs_op, rel)
                    + self.regularizer.forward_dynamic(chunked(rhs_pos, None), chunked(lhs_pos, lhs_op), lhs_op, rel))

    def forward_ranks(self, edges: EdgeList, uniform_negs=None, *, loss: str = "ranking", margin: float = 0.1,
                      relation_weight: float = 1.0, auc_samples: int = 0, auc_seed: int = 0) -> "RankOutput":
        """What ranking evaluation takes from forward() -- the positive scores, the rank
        of every positive among its negatives on either side, the loss -- computed per
        edge on the device without the [B, N] score matrices (pbg_model_ranks;
        reference: eval.py:43-81 over model.py:624-762).  The batch must not be empty."""
        num_pos = len(edges)
        relation_idx, lhs_module, rhs_module = self.resolve(edges)
        if self.num_batch_negs == 0 and self.num_uniform_negs == 0 and not self.relations[relation_idx].all_negs:
            raise ValueError("num_batch_negs and num_uniform_negs cannot both be 0")
        if num_pos == 0:
            raise ValueError("forward_ranks needs at least one edge")
        w_l, w_r = lhs_module.weight, rhs_module.weight
        dev = w_l.device
        spec = self.step_spec(relation_idx, num_pos, w_l.shape[1], loss=loss, margin=float(margin))
        key = ("ranks", relation_idx, num_pos, w_l.data_ptr(), w_r.data_ptr(), loss, float(margin))
        runner = self._runners.get(key)
        if runner is None:
            rhs_op, lhs_op = self.operator_tensors(relation_idx)
            glob = self.global_vectors(relation_idx)
            runner = native.StepRunner(spec, w_l.data, torch.empty(0, device=dev), w_r.data, torch.empty(0, device=dev),
                                       rhs_op, None, lhs_op, None,
                                       global_embs=None if glob is None else (glob[0].data, glob[1].data))
            self._runners[key] = runner
        runner.relation_weights.fill_(float(relation_weight))
        if uniform_negs is None:
            uniform_negs = self.sample_uniform(lhs_module, rhs_module, spec.num_chunks)
        ul, ur = uniform_negs
        lhs = edges.lhs.to_tensor().to(dev).contiguous()
        rhs = edges.rhs.to_tensor().to(dev).contiguous()
        if self.num_dynamic_rels > 0:
            rel = edges.get_relation_type_as_vector().to(dev).contiguous()
        else:
            rel = torch.zeros(1, dtype=torch.int64, device=dev)  # the runner holds this relation's operator only
        weight = edges.weight.to(dev).float().contiguous() if edges.has_weight() else None
        runner._check_ids(lhs, rhs, rel, ul, ur)
        lp, rp, lr, rr, le, hits = runner.ranks(lhs, rhs, rel, ul.contiguous() if ul is not None else None,
                                                ur.contiguous() if ur is not None else None, weight, auc_samples, auc_seed)
        has = (spec.num_negs(self.disable_lhs_negs, w_l.shape[0]) > 0, spec.num_negs(self.disable_rhs_negs, w_r.shape[0]) > 0)
        return RankOutput(lp[0], rp[0], (lr[0], rr[0]), le[0], hits, has)

    def forward(self, edges: EdgeList, uniform_negs=None) -> Tuple[Scores, Optional[FloatTensorType]]:
        """Scores of a batch and the regularizer's value, None without a
        regularizer (model.py:624-762).  `uniform_negs` = (lhs [C,U], rhs [C,U])
        entity indices; drawn with torch.randint when omitted."""
        num_pos = len(edges)
        relation_idx, lhs_module, rhs_module = self.resolve(edges)
        if self.num_batch_negs == 0 and self.num_uniform_negs == 0 and not self.relations[relation_idx].all_negs:
            raise ValueError("num_batch_negs and num_uniform_negs cannot both be 0")
        w_l, w_r = lhs_module.weight, rhs_module.weight
        dim = w_l.shape[1]
        dev = w_l.device
        nl = 0 if self.disable_lhs_negs else None
        if num_pos == 0:
            spec = self.step_spec(relation_idx, 1, dim)
            z = torch.empty((0,), dtype=torch.float32, device=dev)
            return Scores(z, z.clone(), z.new_empty((0, spec.num_negs(self.disable_lhs_negs, w_l.shape[0]))),
                          z.new_empty((0, spec.num_negs(self.disable_rhs_negs, w_r.shape[0])))), None
        spec = self.step_spec(relation_idx, num_pos, dim)
        key = ("fwd", relation_idx, num_pos, w_l.data_ptr(), w_r.data_ptr())
        runner = self._runners.get(key)
        if runner is None:
            rhs_op, lhs_op = self.operator_tensors(relation_idx)
            glob = self.global_vectors(relation_idx)
            runner = native.StepRunner(spec, w_l.data, torch.empty(0, device=dev), w_r.data, torch.empty(0, device=dev),
                                       rhs_op, None, lhs_op, None,
                                       global_embs=None if glob is None else (glob[0].data, glob[1].data))
            self._runners[key] = runner
        if uniform_negs is None:
            uniform_negs = self.sample_uniform(lhs_module, rhs_module, spec.num_chunks)
        ul, ur = uniform_negs
        lhs = edges.lhs.to_tensor().to(dev).contiguous()
        rhs = edges.rhs.to_tensor().to(dev).contiguous()
        if self.num_dynamic_rels > 0:
            rel = edges.get_relation_type_as_vector().to(dev).contiguous()
        else:
            rel = torch.zeros(1, dtype=torch.int64, device=dev)  # the runner holds this relation's operator only
        runner._check_ids(lhs, rhs, rel, ul, ur)  # IndexError, as F.embedding raises it (model.py:60-61)
        lp, rp, ln, rn = runner.forward(lhs, rhs, rel, ul.contiguous() if ul is not None else None,
                                        ur.contiguous() if ur is not None else None)
        reg = None
        if self.regularizer is not None:
            reg = self._regularizer_value(relation_idx, lhs_module, rhs_module, lhs, rhs, rel, spec.chunk_size)
        return Scores(lp[0], rp[0], ln[0], rn[0]), reg
