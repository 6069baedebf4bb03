"""CPU restatement of one PBG training step (test infrastructure only).

Every function cites the reference lines it follows.  The tensor ops are
issued in the reference's order so that fp32 rounding stays comparable, and
uniform-negative indices are INPUTS (the reference draws them with
torch.randint inside the model, model.py:70-75), so that the oracle and the
GPU path can be fed identical negatives.
"""
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import torch
import torch.nn.functional as F

OPERATOR_NAMES = ("none", "diagonal", "translation", "linear", "affine", "complex_diagonal")
COMPARATOR_NAMES = ("dot", "cos", "l2", "squared_l2")
LOSS_NAMES = ("ranking", "logistic", "softmax")


@dataclass
class StepConfig:
    """The fields of the reference's ConfigSchema that parameterise the step
    (config.py:115-347): operator / comparator / loss_fn / margin /
    num_batch_negs / num_uniform_negs / disable_*_negs / dynamic_relations /
    lr / relation_lr, plus per-relation weights (RelationSchema.weight)."""

    dim: int
    operator: str = "none"
    comparator: str = "dot"
    loss: str = "ranking"
    margin: float = 0.1
    num_batch_negs: int = 50
    num_uniform_negs: int = 50
    disable_lhs_negs: bool = False
    disable_rhs_negs: bool = False
    dynamic: bool = False
    num_relations: int = 1
    lr: float = 0.1
    relation_lr: Optional[float] = None
    relation_weights: Sequence[float] = field(default_factory=lambda: [1.0])
    # config.py:221-230: coefficient of the N3 regularizer (the only one registered,
    # regularizers.py:51); 0 = none (model.py:905-909)
    regularization_coef: float = 0.0
    # config.py:181-188: a learned vector per entity type added to every embedding
    # of the type (model.py:433-441,486-492); standard relations only
    global_emb: bool = False
    # config.py:173-180: rows are looked up with F.embedding(max_norm=...), which first
    # renormalises them in the table (model.py:61); None = off
    max_norm: Optional[float] = None
    # config.py:197-207: the first coordinate of every embedding is a bias: it is kept out of
    # the comparator and added to the score (BiasedComparator, model.py:306-344,902-903)
    bias: bool = False
    # RelationSchema.all_negs (config.py:123-131): the negatives of an edge are ALL entities of the
    # side's type, in one chunk (model.py:648-650,582-618)
    all_negs: bool = False
    # config.py:496-498 "Use half-precision training (GPU ONLY)": every embedding is cast to
    # float16 once it is prepared for the comparator (model.py:504-505), so the negative scores are
    # float16 products cast back (model.py:827-829) and the gradient of every prepared embedding is a
    # float16 tensor.  The reference only casts on a CUDA device; here the same statements run on
    # the CPU's Half tensors.
    half_precision: bool = False

    def chunking(self, num_pos: int) -> Tuple[int, int, str]:
        """(chunk_size, num_chunks, mode) as model.py:648-656 and :787."""
        if self.all_negs:
            return num_pos, (1 if num_pos > 0 else 0), "all"
        if self.num_batch_negs == 0:
            chunk = min(self.num_uniform_negs, num_pos)
            mode = "uniform"
        else:
            chunk = min(self.num_batch_negs, num_pos)
            mode = "batch_uniform"
        if num_pos == 0 or chunk == 0:
            return chunk, 0, mode
        return chunk, (num_pos - 1) // chunk + 1, mode


# --------------------------------------------------------------------------
# operators (operators.py:49-157 static, :197-338 dynamic)
# --------------------------------------------------------------------------

def init_operator_params(name: str, dim: int, num_ops: int) -> Dict[str, torch.Tensor]:
    """Initial parameters with a leading [num_ops] axis (operators.py:62,76,
    90,137-138 and :215,234,255-257,315-316).  Standard mode keeps one
    operator object per relation; stacking them changes nothing because a
    relation with a zero gradient is left untouched by Adagrad."""
    if name == "none":
        return {}
    if name == "diagonal":
        return {"diagonal": torch.ones(num_ops, dim)}
    if name == "translation":
        return {"translation": torch.zeros(num_ops, dim)}
    if name == "linear":
        return {"linear_transformation": torch.eye(dim).repeat(num_ops, 1, 1)}
    if name == "affine":  # operators.py:106-107, 276-279
        return {"linear_transformation": torch.eye(dim).repeat(num_ops, 1, 1), "translation": torch.zeros(num_ops, dim)}
    if name == "complex_diagonal":
        if dim % 2 != 0:
            raise ValueError(
                "Need even dimension as 1st half is real and 2nd half is imaginary coordinates"
            )
        return {"real": torch.ones(num_ops, dim // 2), "imag": torch.zeros(num_ops, dim // 2)}
    raise NotImplementedError(f"Unknown operator {name}")


def apply_operator(
    name: str,
    embs: torch.Tensor,
    params: Dict[str, torch.Tensor],
    rel,
) -> torch.Tensor:
    """y = op_rel(x) on the last axis.  ``rel`` is an int (one operator for
    every row: operators.py:53-157) or a LongTensor shaped like
    embs.shape[:-1] (one operator per row: operators.py:200-338)."""
    dim = embs.shape[-1]
    if name == "none":
        return embs
    pick = (lambda p: p[rel])
    if name == "diagonal":
        return pick(params["diagonal"]) * embs
    if name == "translation":
        return embs + pick(params["translation"])
    if name == "linear":
        mat = pick(params["linear_transformation"])
        return torch.matmul(mat, embs.unsqueeze(-1)).squeeze(-1)
    if name == "affine":  # operators.py:109-115, 283-293
        mat = pick(params["linear_transformation"])
        return torch.matmul(mat, embs.unsqueeze(-1)).squeeze(-1) + pick(params["translation"])
    if name == "complex_diagonal":
        half = dim // 2
        real_a, imag_a = embs[..., :half], embs[..., half:]
        real_b, imag_b = pick(params["real"]), pick(params["imag"])
        prod = torch.empty_like(embs)
        prod[..., :half] = real_a * real_b - imag_a * imag_b
        prod[..., half:] = real_a * imag_b + imag_a * real_b
        return prod
    raise NotImplementedError(f"Unknown operator {name}")


# --------------------------------------------------------------------------
# comparators (model.py:159-278)
# --------------------------------------------------------------------------

def comparator_prepare(name: str, embs: torch.Tensor) -> torch.Tensor:
    """model.py:161-162 (dot), :187-192 (cos), :251-252 (l2), :283-284 (squared_l2)."""
    if name == "cos":
        norm = embs.norm(2, dim=-1)
        return embs * norm.reciprocal().unsqueeze(-1)
    if name in ("dot", "l2", "squared_l2"):
        return embs
    raise NotImplementedError(f"Unknown comparator {name}")


def biased_prepare(name: str, embs: torch.Tensor) -> torch.Tensor:
    """BiasedComparator.prepare (model.py:311-314)."""
    return torch.cat([embs[..., :1], comparator_prepare(name, embs[..., 1:])], dim=-1)


def _f32(x: torch.Tensor) -> torch.Tensor:
    """The reference's ``.float()`` casts (model.py:177,268,827-829); float64
    inputs are let through so that tests can take finite differences."""
    return x if x.dtype == torch.float64 else x.float()


def _all_pairs_squared_l2(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """model.py:215-236: ||a||^2 - 2ab + ||b||^2 through baddbmm."""
    a_squared = a.norm(dim=-1).pow(2)
    b_squared = b.norm(dim=-1).pow(2)
    return torch.baddbmm(b_squared.unsqueeze(-2), a, b.transpose(-2, -1), alpha=-2).add_(
        a_squared.unsqueeze(-1)
    )


def _all_pairs_l2(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """model.py:239-246: the above clamped at 1e-30, square-rooted."""
    return _all_pairs_squared_l2(a, b).clamp_min_(1e-30).sqrt_()


def comparator_scores(
    name: str,
    lhs_pos: torch.Tensor,
    rhs_pos: torch.Tensor,
    lhs_neg: torch.Tensor,
    rhs_neg: torch.Tensor,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(pos[C,P], lhs_neg_scores[C,P,Ln] = rhs_pos x lhs_neg,
    rhs_neg_scores[C,P,Rn] = lhs_pos x rhs_neg); model.py:164-182, 194-212,
    254-278, 286-305.  Note the cross pairing of the negative scores."""
    if lhs_pos.dim() != 3 or rhs_pos.shape != lhs_pos.shape:
        raise TypeError("Shape doesn't match")
    c, p, d = lhs_pos.shape
    if lhs_neg.dim() != 3 or lhs_neg.shape[0] != c or lhs_neg.shape[2] != d:
        raise TypeError("Shape doesn't match")
    if rhs_neg.dim() != 3 or rhs_neg.shape[0] != c or rhs_neg.shape[2] != d:
        raise TypeError("Shape doesn't match")
    if name in ("dot", "cos"):
        pos = (_f32(lhs_pos) * _f32(rhs_pos)).sum(-1)
        lneg = torch.bmm(rhs_pos, lhs_neg.transpose(-1, -2))
        rneg = torch.bmm(lhs_pos, rhs_neg.transpose(-1, -2))
        return pos, lneg, rneg
    if name == "l2":
        pos = (_f32(lhs_pos) - _f32(rhs_pos)).pow(2).sum(dim=-1).clamp_min(1e-30).sqrt().neg()
        lneg = _all_pairs_l2(rhs_pos, lhs_neg).neg()
        rneg = _all_pairs_l2(lhs_pos, rhs_neg).neg()
        return pos, lneg, rneg
    if name == "squared_l2":
        pos = (_f32(lhs_pos) - _f32(rhs_pos)).pow(2).sum(dim=-1).neg()
        lneg = _all_pairs_squared_l2(rhs_pos, lhs_neg).neg()
        rneg = _all_pairs_squared_l2(lhs_pos, rhs_neg).neg()
        return pos, lneg, rneg
    raise NotImplementedError(f"Unknown comparator {name}")


def biased_scores(name, lhs_pos, rhs_pos, lhs_neg, rhs_neg):
    """BiasedComparator.forward (model.py:316-344): the base comparator on the
    coordinates after the first, plus the biases of the two rows of a pair."""
    pos, lneg, rneg = comparator_scores(name, lhs_pos[..., 1:], rhs_pos[..., 1:], lhs_neg[..., 1:], rhs_neg[..., 1:])
    lhs_pos_bias = lhs_pos[..., 0]
    rhs_pos_bias = rhs_pos[..., 0]
    pos = pos + lhs_pos_bias + rhs_pos_bias
    lneg = lneg + rhs_pos_bias.unsqueeze(-1) + lhs_neg[..., 0].unsqueeze(-2)
    rneg = rneg + lhs_pos_bias.unsqueeze(-1) + rhs_neg[..., 0].unsqueeze(-2)
    return pos, lneg, rneg


# --------------------------------------------------------------------------
# losses (losses.py:53-161)
# --------------------------------------------------------------------------

def loss_value(
    name: str,
    pos: torch.Tensor,
    neg: torch.Tensor,
    weight: Optional[torch.Tensor],
    margin: float = 0.1,
) -> torch.Tensor:
    num_pos = pos.shape[0]
    if pos.dim() != 1 or neg.dim() != 2 or neg.shape[0] != num_pos:
        raise TypeError("Shape doesn't match")
    num_neg = neg.shape[1]
    if name == "logistic":  # losses.py:55-82
        neg_weight = 1 / num_neg if num_neg > 0 else 0
        pos_loss = F.binary_cross_entropy_with_logits(
            pos, pos.new_ones(()).expand(num_pos), reduction="sum", weight=weight
        )
        neg_loss = F.binary_cross_entropy_with_logits(
            neg,
            neg.new_zeros(()).expand(num_pos, num_neg),
            reduction="sum",
            weight=weight.unsqueeze(-1) if weight is not None else None,
        )
        return pos_loss + neg_weight * neg_loss
    if name == "ranking":  # losses.py:91-124
        if num_pos == 0 or num_neg == 0:
            return torch.zeros((), requires_grad=True)
        per = F.margin_ranking_loss(
            neg,
            pos.unsqueeze(1),
            target=pos.new_full((1, 1), -1, dtype=torch.float),
            margin=margin,
            reduction="none",
        )
        if weight is not None:
            per = per * weight.unsqueeze(-1)
        return per.sum()
    if name == "softmax":  # losses.py:129-161
        if num_pos == 0 or num_neg == 0:
            return torch.zeros((), requires_grad=True)
        scores = torch.cat([pos.unsqueeze(1), neg.logsumexp(dim=1, keepdim=True)], dim=1)
        per = F.cross_entropy(scores, pos.new_zeros((num_pos,), dtype=torch.long), reduction="none")
        if weight is not None:
            per = per * weight
        return per.sum()
    raise NotImplementedError(f"Unknown loss {name}")


# --------------------------------------------------------------------------
# N3 regularizer (regularizers.py:51-97) with the operators' hooks
# (operators.py:39-43,55-56,69-70,83-84,151-157 static; :185-191,206-209,225-228,
# 246-249,332-338 dynamic)
# --------------------------------------------------------------------------

def _embs_for_reg(operator: str, embs: torch.Tensor) -> torch.Tensor:
    """prepare_embs_for_reg: the modulus of each complex coordinate for
    complex_diagonal (operators.py:154-157), |x| otherwise (operators.py:42-43)."""
    if operator == "complex_diagonal":
        h = embs.shape[-1] // 2
        real, imag = embs[..., :h], embs[..., h:]
        return torch.sqrt(real ** 2 + imag ** 2)
    return embs.abs()


def _params_for_reg(operator: str, params: Optional[Dict[str, torch.Tensor]], rel) -> Optional[torch.Tensor]:
    """get_operator_params_for_reg of the operator of relation `rel` (an int:
    operators.py:55-56,69-70,83-84,151-152) or of the operators of the edges
    (LongTensor[B]: operators.py:206-209,225-228,246-249,332-333)."""
    if operator == "none":
        return None
    if operator == "diagonal":
        return params["diagonal"][rel].abs()
    if operator == "translation":
        return params["translation"][rel].abs()
    if operator == "complex_diagonal":
        return torch.sqrt(params["real"][rel] ** 2 + params["imag"][rel] ** 2)
    raise NotImplementedError("Regularizer not implemented for this operator")  # operators.py:40,188


def n3_regularizer(cfg: StepConfig, src_pos: torch.Tensor, dst_pos: torch.Tensor, rel, op_params) -> torch.Tensor:
    """N3Regularizer.forward (standard relations, regularizers.py:82-97) or
    forward_dynamic (regularizers.py:66-80).  src_pos / dst_pos are the chunked
    [C, P, D] positives after operator and comparator.prepare, as
    forward_direction_agnostic passes them (model.py:784-785,800-801,846-854), so
    `len(src_pos)` in the standard branch is the number of CHUNKS."""
    total = 0
    params = _params_for_reg(cfg.operator, op_params, rel)
    if params is not None:
        if isinstance(rel, int):
            total = total + torch.sum(params ** 3) * len(src_pos)
        else:
            total = total + torch.sum(params ** 3)
    for x in (src_pos, dst_pos):
        total = total + torch.sum(_embs_for_reg(cfg.operator, x) ** 3)
    return total * cfg.regularization_coef


# --------------------------------------------------------------------------
# the model forward (model.py:478-856)
# --------------------------------------------------------------------------

@dataclass
class Scores:
    lhs_pos: torch.Tensor
    rhs_pos: torch.Tensor
    lhs_neg: torch.Tensor
    rhs_neg: torch.Tensor
    reg: Optional[torch.Tensor] = None  # the second value MultiRelationEmbedder.forward returns


def _adjust(cfg: StepConfig, embs, rel, op_params, glob=None) -> torch.Tensor:
    """model.py:478-506: global embedding of the entity
    type (``glob``, None = disabled), operator, comparator.prepare.
    ``op_params is None`` means "no operator"."""
    if glob is not None:
        if not isinstance(rel, int):
            raise RuntimeError("Cannot have global embs with dynamic rels")  # model.py:488-489
        embs = embs + glob
    if op_params is not None:
        embs = apply_operator(cfg.operator, embs, op_params, rel)
    embs = (biased_prepare if cfg.bias else comparator_prepare)(cfg.comparator, embs)
    if cfg.half_precision and embs.dtype == torch.float32:  # model.py:504-505 (without its is_cuda condition)
        embs = embs.half()
    return embs


def _direction_agnostic(
    cfg: StepConfig,
    num_pos: int,
    src_pos: torch.Tensor,
    dst_pos: torch.Tensor,
    src_uniform: Optional[torch.Tensor],
    dst_uniform: Optional[torch.Tensor],
    rel,
    dst_op_params,
    chunk_size: int,
    src_method: str,
    dst_method: str,
    src_glob=None,
    dst_glob=None,
    src_ids=None,
    dst_ids=None,
):
    """model.py:764-856.  ``src_uniform`` / ``dst_uniform`` are the raw rows
    of the uniformly sampled entities, [C,U,D] (model.py:544,550); in mode
    "all" they are the side's whole table as [1,E,D] and ``src_ids`` /
    ``dst_ids`` the positives' entities, whose own columns are masked."""
    dim = src_pos.shape[-1]
    src_pos = _adjust(cfg, src_pos, rel, None, src_glob)
    dst_pos = _adjust(cfg, dst_pos, rel, dst_op_params, dst_glob)
    num_chunks = (num_pos - 1) // chunk_size + 1
    pad = num_chunks * chunk_size - num_pos
    if pad > 0:
        src_pos = torch.cat((src_pos, src_pos.new_zeros(()).expand(pad, dim)), dim=0)
        dst_pos = torch.cat((dst_pos, dst_pos.new_zeros(()).expand(pad, dim)), dim=0)
    src_pos = src_pos.view(num_chunks, chunk_size, dim)
    dst_pos = dst_pos.view(num_chunks, chunk_size, dim)
    last = num_pos - (num_chunks - 1) * chunk_size

    def negatives(pos_embs, uniform, method, op_params, glob):
        # model.py:508-622 (NONE / UNIFORM / BATCH_UNIFORM branches)
        masked_batch = False
        if method == "none":
            neg = pos_embs.new_empty((num_chunks, 0, dim))
        elif method == "uniform":
            neg = _adjust(cfg, uniform, rel_for_uniform, op_params, glob)
        elif method == "batch_uniform":
            neg = pos_embs
            if uniform is not None and uniform.shape[1] > 0:
                neg = torch.cat([pos_embs, _adjust(cfg, uniform, rel_for_uniform, op_params, glob)], dim=1)
            masked_batch = True
        elif method == "all":  # model.py:582-618: get_all_entities().expand(num_chunks, -1, dim)
            neg = _adjust(cfg, uniform.expand(num_chunks, -1, dim), rel_for_uniform, op_params, glob)
        else:
            raise NotImplementedError(method)
        return neg, masked_batch

    # The operator is only ever applied to uniform negatives in standard mode,
    # where rel is an int; dynamic mode passes no operator for the negatives.
    rel_for_uniform = rel
    src_neg, src_masked = negatives(src_pos, src_uniform, src_method, None, src_glob)
    dst_neg, dst_masked = negatives(dst_pos, dst_uniform, dst_method, dst_op_params, dst_glob)

    pos_scores, src_neg_scores, dst_neg_scores = (biased_scores if cfg.bias else comparator_scores)(
        cfg.comparator, src_pos, dst_pos, src_neg, dst_neg
    )
    pos_scores = _f32(pos_scores)
    src_neg_scores = _f32(src_neg_scores)
    dst_neg_scores = _f32(dst_neg_scores)

    idx = torch.arange(chunk_size, dtype=torch.long)
    for scores, masked in ((src_neg_scores, src_masked), (dst_neg_scores, dst_masked)):
        if masked:  # model.py:566-580 and :836-839
            scores[: num_chunks - 1, idx, idx] = -1e9
            scores[-1, idx[:last], idx[:last]] = -1e9
            scores[-1, :last, last:chunk_size] = -1e9
    for scores, method, ids in ((src_neg_scores, src_method, src_ids), (dst_neg_scores, dst_method, dst_ids)):
        if method == "all":  # model.py:596-618: ignore_mask[i, pos_input[i]] (one chunk of num_pos rows)
            scores[0, torch.arange(num_pos), ids] = -1e9

    pos_scores = pos_scores.flatten(0, 1)[:num_pos]
    src_neg_scores = src_neg_scores.flatten(0, 1)[:num_pos]
    dst_neg_scores = dst_neg_scores.flatten(0, 1)[:num_pos]
    reg = None
    if cfg.regularization_coef != 0:  # model.py:845-854
        reg = n3_regularizer(cfg, src_pos, dst_pos, rel, dst_op_params)
    return pos_scores, src_neg_scores, dst_neg_scores, reg


def model_forward(
    cfg: StepConfig,
    lhs_pos: torch.Tensor,
    rhs_pos: torch.Tensor,
    lhs_uniform: Optional[torch.Tensor],
    rhs_uniform: Optional[torch.Tensor],
    rel,
    lhs_op_params: Optional[Dict[str, torch.Tensor]],
    rhs_op_params: Optional[Dict[str, torch.Tensor]],
    glob_lhs: Optional[torch.Tensor] = None,
    glob_rhs: Optional[torch.Tensor] = None,
    lhs_ids: Optional[torch.Tensor] = None,
    rhs_ids: Optional[torch.Tensor] = None,
) -> Scores:
    """MultiRelationEmbedder.forward (model.py:624-762) on already gathered
    rows.  lhs_pos/rhs_pos: [B,D] raw rows; *_uniform: [C,U,D] raw rows of the
    uniform negatives (None when U == 0 or the side is disabled); rel: int in
    standard mode, LongTensor[B] in dynamic mode.  With cfg.all_negs the
    *_uniform are the whole tables as [1,E,D] and lhs_ids / rhs_ids the edges'
    entities."""
    num_pos = lhs_pos.shape[0]
    chunk_size, _, mode = cfg.chunking(num_pos)
    lhs_method = "none" if cfg.disable_lhs_negs else mode
    rhs_method = "none" if cfg.disable_rhs_negs else mode
    if not cfg.dynamic:
        if lhs_op_params:
            raise RuntimeError(
                "In non-dynamic relation mode there should be only a right-hand side operator"
            )
        if not isinstance(rel, int):
            raise TypeError("All positive pairs must come from the same relation")
        pos, lneg, rneg, reg = _direction_agnostic(
            cfg, num_pos, lhs_pos, rhs_pos, lhs_uniform, rhs_uniform, rel,
            rhs_op_params if cfg.operator != "none" else None,
            chunk_size, lhs_method, rhs_method, glob_lhs, glob_rhs, lhs_ids, rhs_ids,
        )
        return Scores(pos, pos, lneg, rneg, reg)
    if isinstance(rel, int):
        raise TypeError("Need relation for each positive pair")
    if glob_lhs is not None or glob_rhs is not None:
        raise RuntimeError("Cannot have global embs with dynamic rels")  # model.py:488-489
    # model.py:721-754: forward edges (operator on rhs, negatives on lhs),
    # then reverse edges (operator on lhs, negatives on rhs).
    lpos, lneg, _, l_reg = _direction_agnostic(
        cfg, num_pos, lhs_pos, rhs_pos, lhs_uniform, None, rel,
        rhs_op_params if cfg.operator != "none" else None,
        chunk_size, lhs_method, "none", src_ids=lhs_ids,
    )
    rpos, rneg, _, r_reg = _direction_agnostic(
        cfg, num_pos, rhs_pos, lhs_pos, rhs_uniform, None, rel,
        lhs_op_params if cfg.operator != "none" else None,
        chunk_size, rhs_method, "none", src_ids=rhs_ids,
    )
    reg = None if l_reg is None or r_reg is None else l_reg + r_reg  # model.py:755-758
    return Scores(lpos, rpos, lneg, rneg, reg)


# --------------------------------------------------------------------------
# optimizers (row_adagrad.py:80-107, async_adagrad.py:51-85)
# --------------------------------------------------------------------------

def row_adagrad_sparse(weight: torch.Tensor, state_sum: torch.Tensor, grad: torch.Tensor, lr: float) -> None:
    """row_adagrad.py:80-96 on a sparse COO gradient, in place."""
    if grad._indices().numel() == 0:
        return
    grad = grad.coalesce()
    idx = grad._indices()[0]
    vals = grad._values()
    local_g = state_sum[idx]
    delta = (vals * vals).mean(1)
    state_sum.index_add_(0, idx, delta)
    local_g += delta
    std = local_g.sqrt_().add_(1e-10).unsqueeze(1)
    weight.index_add_(0, idx, -lr * vals / std)


def row_adagrad_dense(weight: torch.Tensor, state_sum: torch.Tensor, grad: torch.Tensor, lr: float) -> None:
    """row_adagrad.py:97-107, in place."""
    local_g = state_sum.clone()
    delta = (grad * grad).mean(1)
    state_sum += delta
    local_g += delta
    std = local_g.sqrt().add_(1e-10)
    weight.addcdiv_(grad, std.unsqueeze(1), value=-lr)


def async_adagrad_dense(param: torch.Tensor, state_sum: torch.Tensor, grad: torch.Tensor, lr: float, eps: float = 1e-10) -> None:
    """async_adagrad.py:75-85 with lr_decay = 0, in place."""
    local_g = state_sum.clone()
    delta = grad * grad
    state_sum.add_(delta)
    local_g += delta
    std = local_g.sqrt().add_(eps)
    param.addcdiv_(grad, std, value=-lr)


# --------------------------------------------------------------------------
# one training step (train_cpu.py:86-112 + batching.py:139-150)
# --------------------------------------------------------------------------

@dataclass
class TrainState:
    """Tables and optimizer state the step mutates.  ``w_rhs is w_lhs`` when
    both sides share one entity type (model.py:454-472 wraps the same
    Parameter for both sides)."""

    w_lhs: torch.Tensor
    g_lhs: torch.Tensor
    w_rhs: torch.Tensor
    g_rhs: torch.Tensor
    lhs_op: Dict[str, torch.Tensor] = field(default_factory=dict)
    rhs_op: Dict[str, torch.Tensor] = field(default_factory=dict)
    lhs_op_sum: Dict[str, torch.Tensor] = field(default_factory=dict)
    rhs_op_sum: Dict[str, torch.Tensor] = field(default_factory=dict)
    # global embeddings of the two sides' entity types and their AsyncAdagrad sums
    # (None = disabled); the same tensors on both sides when the sides share a type
    glob_lhs: Optional[torch.Tensor] = None
    glob_rhs: Optional[torch.Tensor] = None
    glob_lhs_sum: Optional[torch.Tensor] = None
    glob_rhs_sum: Optional[torch.Tensor] = None

    @property
    def shared(self) -> bool:
        return self.w_lhs is self.w_rhs


def make_state(cfg: StepConfig, w_lhs: torch.Tensor, w_rhs: Optional[torch.Tensor] = None) -> TrainState:
    shared = w_rhs is None
    g_lhs = torch.zeros(w_lhs.shape[0])
    st = TrainState(
        w_lhs=w_lhs,
        g_lhs=g_lhs,
        w_rhs=w_lhs if shared else w_rhs,
        g_rhs=g_lhs if shared else torch.zeros(w_rhs.shape[0]),
    )
    st.rhs_op = init_operator_params(cfg.operator, cfg.dim, cfg.num_relations)
    st.rhs_op_sum = {k: torch.zeros_like(v) for k, v in st.rhs_op.items()}
    if cfg.dynamic:
        st.lhs_op = init_operator_params(cfg.operator, cfg.dim, cfg.num_relations)
        st.lhs_op_sum = {k: torch.zeros_like(v) for k, v in st.lhs_op.items()}
    if cfg.global_emb:  # model.py:433-439: zeros, one vector per entity type
        st.glob_lhs, st.glob_lhs_sum = torch.zeros(cfg.dim), torch.zeros(cfg.dim)
        if shared:
            st.glob_rhs, st.glob_rhs_sum = st.glob_lhs, st.glob_lhs_sum
        else:
            st.glob_rhs, st.glob_rhs_sum = torch.zeros(cfg.dim), torch.zeros(cfg.dim)
    return st


@dataclass
class StepOutput:
    loss: float
    violators_lhs: int
    violators_rhs: int
    count: int
    scores: Optional[Scores] = None
    reg: float = 0.0


@dataclass
class StepGrads:
    """Gradients of one batch, before any update is applied."""

    sparse_lhs: Optional[torch.Tensor]  # sparse COO on w_lhs (also carries rhs grads when shared)
    sparse_rhs: Optional[torch.Tensor]
    lhs_op: Dict[str, torch.Tensor]
    rhs_op: Dict[str, torch.Tensor]
    glob_lhs: Optional[torch.Tensor] = None  # also carries the rhs side's sum when the sides share a type
    glob_rhs: Optional[torch.Tensor] = None


def forward_backward(
    cfg: StepConfig,
    st: TrainState,
    lhs: torch.Tensor,
    rhs: torch.Tensor,
    rel,
    uniform_lhs: Optional[torch.Tensor],
    uniform_rhs: Optional[torch.Tensor],
    weight: Optional[torch.Tensor] = None,
    keep_scores: bool = False,
) -> Tuple[StepOutput, StepGrads]:
    """zero_grad -> forward -> calc_loss -> stats -> backward
    (train_cpu.py:89-105).  uniform_*: LongTensor[C,U] entity indices."""
    w_l = st.w_lhs.detach().requires_grad_(True)
    w_r = w_l if st.shared else st.w_rhs.detach().requires_grad_(True)
    lhs_op = {k: v.detach().requires_grad_(True) for k, v in st.lhs_op.items()}
    rhs_op = {k: v.detach().requires_grad_(True) for k, v in st.rhs_op.items()}

    # (with max_norm the tables themselves change here, before anything is computed: model.py:61)
    lhs_pos = F.embedding(lhs, w_l, max_norm=cfg.max_norm, sparse=True)
    rhs_pos = F.embedding(rhs, w_r, max_norm=cfg.max_norm, sparse=True)
    lhs_u = (
        F.embedding(uniform_lhs, w_l, max_norm=cfg.max_norm, sparse=True)
        if uniform_lhs is not None and not cfg.disable_lhs_negs and uniform_lhs.numel() > 0
        else None
    )
    rhs_u = (
        F.embedding(uniform_rhs, w_r, max_norm=cfg.max_norm, sparse=True)
        if uniform_rhs is not None and not cfg.disable_rhs_negs and uniform_rhs.numel() > 0
        else None
    )
    if cfg.all_negs:  # module.get_all_entities() (model.py:66-68,584): every row, looked up like the others
        lhs_u = None if cfg.disable_lhs_negs else F.embedding(
            torch.arange(w_l.shape[0]).unsqueeze(0), w_l, max_norm=cfg.max_norm, sparse=True)
        rhs_u = None if cfg.disable_rhs_negs else F.embedding(
            torch.arange(w_r.shape[0]).unsqueeze(0), w_r, max_norm=cfg.max_norm, sparse=True)
    glob_l = glob_r = None
    if st.glob_lhs is not None:
        glob_l = st.glob_lhs.detach().requires_grad_(True)
        glob_r = glob_l if st.glob_rhs is st.glob_lhs else st.glob_rhs.detach().requires_grad_(True)
    scores = model_forward(cfg, lhs_pos, rhs_pos, lhs_u, rhs_u, rel, lhs_op or None, rhs_op or None, glob_l, glob_r,
                           lhs, rhs)

    # batching.py:139-150
    lhs_loss = loss_value(cfg.loss, scores.lhs_pos, scores.lhs_neg, weight, cfg.margin)
    rhs_loss = loss_value(cfg.loss, scores.rhs_pos, scores.rhs_neg, weight, cfg.margin)
    relation = rel if isinstance(rel, int) else 0
    loss = cfg.relation_weights[relation] * (lhs_loss + rhs_loss)

    out = StepOutput(
        loss=float(loss.detach()),
        violators_lhs=int((scores.lhs_neg > scores.lhs_pos.unsqueeze(1)).sum()),
        violators_rhs=int((scores.rhs_neg > scores.rhs_pos.unsqueeze(1)).sum()),
        count=int(lhs.shape[0]),
        scores=Scores(
            scores.lhs_pos.detach(), scores.rhs_pos.detach(),
            scores.lhs_neg.detach(), scores.rhs_neg.detach(),
        ) if keep_scores else None,
        reg=float(scores.reg.detach()) if scores.reg is not None else 0.0,
    )
    if scores.reg is not None:  # train_cpu.py:102-105
        (loss + scores.reg).backward()
    else:
        loss.backward()
    grads = StepGrads(
        sparse_lhs=w_l.grad,
        sparse_rhs=None if st.shared else w_r.grad,
        lhs_op={k: (v.grad if v.grad is not None else torch.zeros_like(v)) for k, v in lhs_op.items()},
        rhs_op={k: (v.grad if v.grad is not None else torch.zeros_like(v)) for k, v in rhs_op.items()},
        glob_lhs=None if glob_l is None else (glob_l.grad if glob_l.grad is not None else torch.zeros_like(glob_l)),
        glob_rhs=None if glob_r is None or glob_r is glob_l else
        (glob_r.grad if glob_r.grad is not None else torch.zeros_like(glob_r)),
    )
    return out, grads


def apply_grads(cfg: StepConfig, st: TrainState, grads: StepGrads) -> None:
    """model_optimizer.step then the per-entity RowAdagrad steps
    (train_cpu.py:106-110; lr choice train_cpu.py:224-228)."""
    rel_lr = cfg.relation_lr if cfg.relation_lr is not None else cfg.lr
    with torch.no_grad():
        for params, sums, g in (
            (st.lhs_op, st.lhs_op_sum, grads.lhs_op),
            (st.rhs_op, st.rhs_op_sum, grads.rhs_op),
        ):
            for name, p in params.items():
                async_adagrad_dense(p, sums[name], g[name], rel_lr)
        # the global embeddings are parameters of the model too (model.py:433-439)
        if grads.glob_lhs is not None:
            async_adagrad_dense(st.glob_lhs, st.glob_lhs_sum, grads.glob_lhs, rel_lr)
        if grads.glob_rhs is not None:
            async_adagrad_dense(st.glob_rhs, st.glob_rhs_sum, grads.glob_rhs, rel_lr)
        if grads.sparse_lhs is not None:
            row_adagrad_sparse(st.w_lhs, st.g_lhs, grads.sparse_lhs, cfg.lr)
        if grads.sparse_rhs is not None:
            row_adagrad_sparse(st.w_rhs, st.g_rhs, grads.sparse_rhs, cfg.lr)


def train_step(cfg, st, lhs, rhs, rel, uniform_lhs, uniform_rhs, weight=None, keep_scores=False) -> StepOutput:
    """Trainer._process_one_batch (train_cpu.py:86-112) for one batch."""
    out, grads = forward_backward(cfg, st, lhs, rhs, rel, uniform_lhs, uniform_rhs, weight, keep_scores)
    apply_grads(cfg, st, grads)
    return out


def train_lockstep(cfg, st, batches: List[tuple], keep_scores: bool = False) -> List[StepOutput]:
    """K HOGWILD workers (train_cpu.py:849-884) in the one interleaving that is
    deterministic: every worker reads the tables, then every worker writes, in
    worker order.  ``batches`` is a list of (lhs, rhs, rel, uniform_lhs,
    uniform_rhs) tuples, one per worker."""
    outs, all_grads = [], []
    for b in batches:
        out, grads = forward_backward(cfg, st, *b, keep_scores=keep_scores)
        outs.append(out)
        all_grads.append(grads)
    for grads in all_grads:
        apply_grads(cfg, st, grads)
    return outs
