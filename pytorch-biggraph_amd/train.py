"""The training batch processor (reference: torchbiggraph/train_cpu.py:74-112,
215-230).  ``Trainer._process_one_batch`` is ONE call into libpbg_hip
(pbg_train_step): forward, loss, statistics, backward, AsyncAdagrad on the
operator parameters and RowAdagrad on the embedding tables."""
from typing import Dict, Iterable, List, Optional, Tuple

import torch
from torch.optim import Optimizer

from . import native
from .async_adagrad import AsyncAdagrad
from .batching import AbstractBatchProcessor
from .edgelist import EdgeList
from .losses import AbstractLossFunction
from .model import MultiRelationEmbedder
from .row_adagrad import RowAdagrad
from .stats import Stats
from .util import DummyOptimizer


def make_optimizer(params: Iterable[torch.nn.Parameter], is_emb: bool, lr: float,
                   relation_lr: Optional[float] = None) -> Optimizer:
    """RowAdagrad for embedding tables, AsyncAdagrad (with relation_lr if given)
    for everything else, DummyOptimizer for nothing (train_cpu.py:215-230)."""
    params = list(params)
    if len(params) == 0:
        return DummyOptimizer()
    if is_emb:
        return RowAdagrad(params, lr=lr)
    return AsyncAdagrad(params, lr=relation_lr if relation_lr is not None else lr)


class Trainer(AbstractBatchProcessor):
    def __init__(self, model_optimizer: Optimizer, loss_fn: AbstractLossFunction, relation_weights: List[float]) -> None:
        super().__init__(loss_fn, relation_weights)
        self.model_optimizer = model_optimizer
        self.unpartitioned_optimizers: Dict[str, Optimizer] = {}
        self.partitioned_optimizers: Dict[Tuple[str, int], Optimizer] = {}
        self._runners: Dict[tuple, native.StepRunner] = {}
        # set to (uniform_lhs [C,U], uniform_rhs [C,U]) to feed the next batch's negatives from outside
        self.next_uniform_negs = None
        # False: ids outside their table are clamped by the kernels instead of raising IndexError
        self.check_ids = True

    def _embedding_optimizer(self, weight: torch.nn.Parameter) -> RowAdagrad:
        for opt in list(self.unpartitioned_optimizers.values()) + list(self.partitioned_optimizers.values()):
            if isinstance(opt, RowAdagrad):
                for group in opt.param_groups:
                    if any(p is weight for p in group["params"]):
                        return opt
        raise RuntimeError("No RowAdagrad optimizer owns the embedding table of this batch")

    def _operator_state(self, params: Dict[str, torch.Tensor], owners) -> Dict[str, torch.Tensor]:
        sums = {}
        for name, owner in owners.items():
            state = self.model_optimizer.state[owner]
            if "sum" not in state:
                raise RuntimeError("The model optimizer holds no Adagrad state for an operator parameter")
            sums[name] = state["sum"]
        return sums

    def _process_one_batch(self, model: MultiRelationEmbedder, batch_edges: EdgeList) -> Stats:
        num_pos = len(batch_edges)
        if num_pos == 0:
            return Stats(loss=0.0, reg=0.0, violators_lhs=0, violators_rhs=0, count=0)
        relation_idx, lhs_module, rhs_module = model.resolve(batch_edges)
        w_l, w_r = lhs_module.weight, rhs_module.weight
        dev = w_l.device
        opt_l, opt_r = self._embedding_optimizer(w_l), self._embedding_optimizer(w_r)
        lr = opt_l.param_groups[0]["lr"]
        rel_lr = self.model_optimizer.param_groups[0]["lr"] if len(self.model_optimizer.param_groups) and \
            self.model_optimizer.param_groups[0]["params"] else lr
        key = (relation_idx, num_pos, w_l.data_ptr(), w_r.data_ptr(), lr, rel_lr)
        runner = self._runners.get(key)
        if runner is None:
            spec = model.step_spec(relation_idx, num_pos, w_l.shape[1], loss=self.loss_fn.loss_name,
                                   margin=self.loss_fn.fused_margin, lr=lr, relation_lr=rel_lr)
            rhs_op, lhs_op = model.operator_tensors(relation_idx)

            def sums(op_module, tensors):
                if not tensors:
                    return {}
                p0, p1 = op_module.fused_params()
                owners = {"p0": p0, "p1": p1} if p1 is not None else {"p0": p0}
                return self._operator_state(tensors, owners)

            rhs_sum = sums(model.rhs_operators[relation_idx], rhs_op)
            lhs_sum = sums(model.lhs_operators[relation_idx], lhs_op) if model.num_dynamic_rels > 0 else {}
            dynamic = model.num_dynamic_rels > 0
            weights = list(self.relation_weights) if dynamic else [self.relation_weights[relation_idx]]
            if dynamic:
                weights = (weights + [1.0] * model.num_dynamic_rels)[:model.num_dynamic_rels]
            rw = torch.tensor(weights, dtype=torch.float32, device=dev)
            glob = model.global_vectors(relation_idx)
            glob_sums = None
            if glob is not None:  # parameters of the model optimizer, like the operators'
                glob_sums = tuple(self._operator_state({}, {"g": p})["g"] for p in glob)
            runner = native.StepRunner(spec, w_l.data, opt_l.state[w_l]["sum"], w_r.data, opt_r.state[w_r]["sum"],
                                       rhs_op, rhs_sum, lhs_op, lhs_sum, relation_weights=rw,
                                       global_embs=None if glob is None else (glob[0].data, glob[1].data),
                                       global_sums=glob_sums)
            self._runners[key] = runner
        negs = self.next_uniform_negs
        self.next_uniform_negs = None
        if negs is None:
            negs = model.sample_uniform(lhs_module, rhs_module, runner.spec.num_chunks)
        ul, ur = negs
        lhs = batch_edges.lhs.to_tensor().to(dev).contiguous()
        rhs = batch_edges.rhs.to_tensor().to(dev).contiguous()
        if model.num_dynamic_rels > 0:
            rel = batch_edges.get_relation_type_as_vector().to(dev).contiguous()
        else:
            rel = torch.zeros(1, dtype=torch.int64, device=dev)
        weight = batch_edges.weight
        if weight is not None:
            weight = weight.to(device=dev, dtype=torch.float32).expand(num_pos).contiguous()
        # An id outside its table raises IndexError here, as F.embedding does in the reference (model.py:60-61);
        # the kernels themselves would clamp it.  The check's synchronisation is one this method has anyway.
        runner.train(lhs, rhs, rel, ul.contiguous() if ul is not None else None,
                     ur.contiguous() if ur is not None else None, weight, check_ids=self.check_ids)
        # the reference reads loss and both violator counts on the host for every batch (train_cpu.py:95-101)
        viol = runner.violators_out[0].tolist()
        return Stats(loss=float(runner.loss_out[0]), reg=float(runner.reg_out[0]), violators_lhs=int(viol[0]), violators_rhs=int(viol[1]),
                     count=num_pos)
