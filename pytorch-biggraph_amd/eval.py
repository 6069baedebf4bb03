"""Ranking evaluation of a batch (reference: torchbiggraph/eval.py:43-86,
util.py:420-428, stats.py:16-17).  The scores come from
MultiRelationEmbedder.forward, i.e. from pbg_model_forward on the GPU; the
metrics are a handful of reductions over [B] and [B, N] tensors."""
from statistics import mean

import torch

from .batching import AbstractBatchProcessor
from .edgelist import EdgeList
from .model import MultiRelationEmbedder, Scores
from .stats import Stats


def average_of_sums(*tensors: torch.Tensor) -> float:
    """stats.py:16-17."""
    return mean(t.sum().item() for t in tensors)


def compute_randomized_auc(pos_: torch.Tensor, neg_: torch.Tensor, num_samples: int) -> float:
    """Probability that a randomly chosen positive scores higher than a randomly
    chosen negative, from num_samples random pairs (util.py:420-428)."""
    pos_, neg_ = pos_.reshape(-1), neg_.reshape(-1)
    dev = pos_.device
    diff = (pos_[torch.randint(len(pos_), (num_samples,), device=dev)]
            > neg_[torch.randint(len(neg_), (num_samples,), device=dev)])
    return float(diff.float().mean())


def ranking_stats(sides, loss: float, count: int) -> Stats:
    """The sums RankingEvaluator reports for `count` edges (eval.py:57-81).
    sides: (pos [n], neg [n, N]) per side; a side without negatives is skipped.
    Rank = 1 + number of negatives scoring at least as high as the positive."""
    ranks, aucs = [], []
    for pos, neg in sides:
        if neg.nelement() > 0:
            ranks.append((neg >= pos.unsqueeze(1)).sum(1) + 1)
            aucs.append(compute_randomized_auc(pos, neg, count))
    return Stats(
        loss=float(loss),
        pos_rank=average_of_sums(*ranks),
        mrr=average_of_sums(*(rank.float().reciprocal() for rank in ranks)),
        r1=average_of_sums(*(rank.le(1) for rank in ranks)),
        r10=average_of_sums(*(rank.le(10) for rank in ranks)),
        r50=average_of_sums(*(rank.le(50) for rank in ranks)),
        auc=count * sum(aucs) / len(aucs),  # averaged over count at the end
        count=count,
    )


def ranking_stats_from_ranks(ranks, loss: float, count: int, auc_hits=None, auc_samples: int = 0) -> Stats:
    """The same sums from per-edge ranks (StepRunner.ranks / pbg_model_ranks), one
    int64 tensor per side that has negatives.  auc_hits[side] of auc_samples random
    (positive, negative) pairs had positive > negative (util.py:420-428)."""
    ranks = [r.reshape(-1) for r in ranks]
    if auc_hits is not None and auc_samples > 0:
        auc = count * sum(float(h) / auc_samples for h in auc_hits) / len(auc_hits)
    else:
        auc = 0.0
    return Stats(
        loss=float(loss),
        pos_rank=average_of_sums(*ranks),
        mrr=average_of_sums(*(rank.float().reciprocal() for rank in ranks)),
        r1=average_of_sums(*(rank.le(1) for rank in ranks)),
        r10=average_of_sums(*(rank.le(10) for rank in ranks)),
        r50=average_of_sums(*(rank.le(50) for rank in ranks)),
        auc=auc,
        count=count,
    )


class RankingEvaluator(AbstractBatchProcessor):
    """eval.py:43-86: rank of each positive among its negatives (ties count
    against the positive), MRR, hits@1/10/50 and a randomized AUC, averaged over
    the sides that have negatives; sums over the batch, to be divided by count."""

    def _process_one_batch(self, model: MultiRelationEmbedder, batch_edges: EdgeList) -> Stats:
        # Without a score filter (the _adjust_scores hook) nothing needs the [B, N] score matrices: ranks,
        # loss and the AUC count come from one call, per edge.
        if type(self)._adjust_scores is RankingEvaluator._adjust_scores and len(batch_edges) > 0:
            count = len(batch_edges)
            kind = batch_edges.get_relation_type_as_scalar() if batch_edges.has_scalar_relation_type() else 0
            out = model.forward_ranks(batch_edges, loss=self.loss_fn.loss_name, margin=self.loss_fn.fused_margin,
                                      relation_weight=float(self.relation_weights[kind]), auc_samples=count,
                                      auc_seed=int(torch.randint(0, 2**62, (1,))))
            sides = [s for s in range(2) if out.has_negs[s]]
            return ranking_stats_from_ranks([out.ranks[s] for s in sides], float(out.loss_edge.sum()), count,
                                            [out.auc_hits[s] for s in sides], count)
        with torch.no_grad():
            scores, _ = model(batch_edges)
        self._adjust_scores(scores, batch_edges)
        loss = self.calc_loss(scores, batch_edges)
        return ranking_stats(((scores.lhs_pos, scores.lhs_neg), (scores.rhs_pos, scores.rhs_neg)), float(loss),
                             len(batch_edges))

    def _adjust_scores(self, scores: Scores, batch_edges: EdgeList) -> None:
        """Hook for a filtered evaluator (eval.py:82-86)."""
