"""Tensor-level wrappers over the C ABI: torch tensors in, device pointers out.

PyTorch is plumbing here (device memory, the current stream); all arithmetic
happens inside libpbg_hip.so.
"""
import ctypes
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from . import _lib
from ._lib import COMPARATOR_CODES, LOSS_CODES, OPERATOR_CODES, StepBuffers, StepDesc, check


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    if t is None:
        return None
    return t.data_ptr()


def _need(t: torch.Tensor, dtype: torch.dtype, name: str) -> torch.Tensor:
    if not t.is_cuda:
        raise TypeError(f"{name} must live on the GPU (there is no CPU path)")
    if t.dtype != dtype:
        raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    return t


def _workspace(nbytes: int, device) -> torch.Tensor:
    return torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)


# ---------------------------------------------------------------------------
def gather_rows(table: torch.Tensor, idx: torch.Tensor, check_bounds: bool = True) -> torch.Tensor:
    """out[i] = table[idx[i]] (SimpleEmbedding.get)."""
    _need(table, torch.float32, "table")
    _need(idx, torch.int64, "idx")
    if table.dim() != 2:
        raise ValueError("table must be 2-dimensional")
    flat = idx.reshape(-1)
    out = torch.empty((flat.shape[0], table.shape[1]), dtype=torch.float32, device=table.device)
    flag = torch.zeros(1, dtype=torch.int32, device=table.device) if check_bounds else None
    check(_lib.lib().pbg_gather_rows(_ptr(table), table.shape[0], table.shape[1], _ptr(flat), flat.shape[0],
                                     _ptr(out), _ptr(flag), _stream()))
    if check_bounds and int(flag.item()) != 0:
        raise IndexError("index out of range in gather_rows")
    return out.view(*idx.shape, table.shape[1])


def embedding_renorm_(table: torch.Tensor, idx: torch.Tensor, max_norm: float) -> None:
    """In the table: every row named in idx with a 2-norm above max_norm is
    scaled to max_norm (torch.embedding_renorm_, the first half of
    F.embedding(max_norm=...), model.py:61)."""
    _need(table, torch.float32, "table")
    _need(idx, torch.int64, "idx")
    flat = idx.reshape(-1).contiguous()
    n, dim = flat.shape[0], table.shape[1]
    if n == 0:
        return
    nbytes = _lib.lib().pbg_embedding_renorm_workspace_bytes(n, dim)
    ws = _workspace(nbytes, table.device)
    check(_lib.lib().pbg_embedding_renorm(_ptr(table), table.shape[0], dim, _ptr(flat), n, float(max_norm), _ptr(ws),
                                          nbytes, _stream()))


def row_adagrad_sparse(weight: torch.Tensor, state_sum: torch.Tensor, idx: torch.Tensor,
                       grad_rows: torch.Tensor, lr: float, workspace: Optional[torch.Tensor] = None) -> None:
    _need(weight, torch.float32, "weight")
    _need(state_sum, torch.float32, "state_sum")
    _need(idx, torch.int64, "idx")
    _need(grad_rows, torch.float32, "grad_rows")
    n = idx.shape[0]
    if grad_rows.shape != (n, weight.shape[1]):
        raise ValueError("grad_rows must be [len(idx), dim]")
    nbytes = _lib.lib().pbg_row_adagrad_sparse_workspace_bytes(n)
    if workspace is None or workspace.numel() < nbytes:
        workspace = _workspace(nbytes, weight.device)
    check(_lib.lib().pbg_row_adagrad_sparse(_ptr(weight), _ptr(state_sum), weight.shape[0], weight.shape[1],
                                            _ptr(idx), _ptr(grad_rows), n, float(lr), _ptr(workspace),
                                            workspace.numel(), _stream()))


def row_adagrad_dense(weight: torch.Tensor, state_sum: torch.Tensor, grad: torch.Tensor, lr: float) -> None:
    _need(weight, torch.float32, "weight")
    _need(state_sum, torch.float32, "state_sum")
    _need(grad, torch.float32, "grad")
    if grad.shape != weight.shape:
        raise ValueError("grad must have the shape of weight")
    check(_lib.lib().pbg_row_adagrad_dense(_ptr(weight), _ptr(state_sum), weight.shape[0], weight.shape[1],
                                           _ptr(grad), float(lr), _stream()))


def async_adagrad_dense(param: torch.Tensor, state_sum: torch.Tensor, grad: torch.Tensor, lr: float,
                        eps: float = 1e-10) -> None:
    _need(param, torch.float32, "param")
    _need(state_sum, torch.float32, "state_sum")
    _need(grad, torch.float32, "grad")
    check(_lib.lib().pbg_async_adagrad_dense(_ptr(param), _ptr(state_sum), _ptr(grad), param.numel(), float(lr),
                                             float(eps), _stream()))


def bmm_nt(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """[batch, m, k] x [batch, n, k]^T -> [batch, m, n] on the matrix cores."""
    _need(a, torch.float32, "a")
    _need(b, torch.float32, "b")
    batch, m, k = a.shape
    n = b.shape[1]
    c = torch.empty((batch, m, n), dtype=torch.float32, device=a.device)
    check(_lib.lib().pbg_gemm_f32(_ptr(a), _ptr(b), _ptr(c), batch, m, n, k, k, k, n, m * k, n * k, m * n, 0, 0,
                                  1.0, 0.0, _stream()))
    return c


def gemm(a, b, c, batch, m, n, k, lda, ldb, ldc, stride_a, stride_b, stride_c, a_kmajor, b_kmajor,
         alpha=1.0, beta=0.0, half=False) -> None:
    """`half`: the operands hold float16 numbers; the product as torch.bmm makes it on Half tensors (pbg_gemm_f16)."""
    fn = _lib.lib().pbg_gemm_f16 if half else _lib.lib().pbg_gemm_f32
    check(fn(_ptr(a), _ptr(b), _ptr(c), batch, m, n, k, lda, ldb, ldc, stride_a, stride_b,
                                  stride_c, int(a_kmajor), int(b_kmajor), float(alpha), float(beta), _stream()))


def sample_uniform_negatives(seed: int, side: int, num_rows: int, shape, device) -> torch.Tensor:
    """The rows a step draws for `side` (0 lhs, 1 rhs) under `seed`, as
    [num_workers, num_chunks, num_uniform_negs] = `shape`."""
    out = torch.empty(tuple(shape), dtype=torch.int64, device=device)
    check(_lib.lib().pbg_sample_uniform_negatives(seed & (2**64 - 1), side, num_rows, out.numel(), _ptr(out), _stream()))
    return out


# ---------------------------------------------------------------------------
def reverse_permutation(perm: torch.Tensor) -> torch.Tensor:
    _need(perm, torch.int64, "perm")
    out = torch.empty_like(perm)
    check(_lib.lib().pbg_reverse_permutation(_ptr(perm), perm.shape[0], _ptr(out), _stream()))
    return out


def shuffle_rows(tensor: torch.Tensor, perm: torch.Tensor, scratch: Optional[torch.Tensor] = None) -> None:
    """In place: row i of `tensor` moves to row perm[i]."""
    n = tensor.shape[0]
    row_bytes = tensor[0].numel() * tensor.element_size() if n > 0 else 0
    if n == 0 or row_bytes == 0:
        return
    nbytes = n * row_bytes
    if scratch is None or scratch.numel() * scratch.element_size() < nbytes:
        scratch = _workspace(nbytes, tensor.device)
    flag = torch.zeros(1, dtype=torch.int32, device=tensor.device)
    check(_lib.lib().pbg_shuffle_rows(_ptr(tensor), n, row_bytes, _ptr(perm), _ptr(scratch), _ptr(flag), _stream()))
    if int(flag.item()) != 0:
        raise ValueError("Permutation has out-of-bound values")


def shuffle_rows_out(tensor: torch.Tensor, perm: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[perm[i]] = tensor[i] into a second buffer (returned): the in-place form without its copy back."""
    if not tensor.is_contiguous():
        raise ValueError("tensor must be contiguous")
    if out is None:
        out = torch.empty_like(tensor)
    n = tensor.shape[0]
    row_bytes = tensor[0].numel() * tensor.element_size() if n > 0 else 0
    if n == 0 or row_bytes == 0:
        return out
    flag = torch.zeros(1, dtype=torch.int32, device=tensor.device)
    check(_lib.lib().pbg_shuffle_rows_out(_ptr(tensor), n, row_bytes, _ptr(perm), _ptr(out), _ptr(flag), _stream()))
    if int(flag.item()) != 0:
        raise ValueError("Permutation has out-of-bound values")
    return out


def randperm(n: int, seed: int, device) -> torch.Tensor:
    out = torch.empty(n, dtype=torch.int64, device=device)
    check(_lib.lib().pbg_randperm(n, seed & (2**64 - 1), _ptr(out), None, 0, _stream()))
    return out


def sub_bucket(lhs_in, rhs_in, rel_in, lhs_perms: Sequence[torch.Tensor], rhs_perms: Sequence[torch.Tensor],
               lhs_part_sizes: Sequence[int], rhs_part_sizes: Sequence[int], num_lhs_parts: int, num_rhs_parts: int,
               dynamic_relations: bool, lhs_out, rhs_out, rel_out) -> torch.Tensor:
    """Returns the device tensor offsets[parts_l * parts_r + 1]."""
    dev = lhs_in.device
    n = rel_in.shape[0]
    num_rel = len(lhs_perms)
    lptr = torch.tensor([p.data_ptr() for p in lhs_perms], dtype=torch.int64, device=dev)
    rptr = torch.tensor([p.data_ptr() for p in rhs_perms], dtype=torch.int64, device=dev)
    lsz = torch.tensor(list(lhs_part_sizes), dtype=torch.int64, device=dev)
    rsz = torch.tensor(list(rhs_part_sizes), dtype=torch.int64, device=dev)
    offsets = torch.empty(num_lhs_parts * num_rhs_parts + 1, dtype=torch.int64, device=dev)
    flag = torch.zeros(1, dtype=torch.int32, device=dev)
    nbytes = _lib.lib().pbg_sub_bucket_workspace_bytes(n)
    ws = _workspace(nbytes, dev)
    check(_lib.lib().pbg_sub_bucket(_ptr(lhs_in), _ptr(rhs_in), _ptr(rel_in), n, num_rel, _ptr(lptr), _ptr(rptr),
                                    _ptr(lsz), _ptr(rsz), num_lhs_parts, num_rhs_parts, int(dynamic_relations),
                                    _ptr(lhs_out), _ptr(rhs_out), _ptr(rel_out), _ptr(offsets), _ptr(flag),
                                    _ptr(ws), ws.numel(), _stream()))
    code = int(flag.item())
    if code == 1:
        raise RuntimeError("rel > numRelations")
    if code == 2:
        raise RuntimeError("entity offset outside its sub-partitions")
    return offsets


# ---------------------------------------------------------------------------
@dataclass
class StepSpec:
    """Host-side description of one training-step configuration."""

    dim: int
    batch_size: int
    num_workers: int = 1
    num_batch_negs: int = 50
    num_uniform_negs: int = 50
    disable_lhs_negs: bool = False
    disable_rhs_negs: bool = False
    operator: str = "none"
    dynamic: bool = False
    num_relations: int = 1
    comparator: str = "dot"
    loss: str = "ranking"
    margin: float = 0.1
    lr: float = 0.1
    relation_lr: Optional[float] = None
    regularization_coef: float = 0.0  # config.regularization_coef of the N3 regularizer; 0 = none
    max_norm: Optional[float] = None  # config.max_norm: looked-up rows are first renormalised in the table
    bias: bool = False  # config.bias: BiasedComparator around the comparator
    # RelationSchema.all_negs: one chunk, every entity of a side's type is a negative (model.py:648-650,582-618)
    all_negs: bool = False
    # config.half_precision: embeddings are float16 numbers from comparator.prepare on (model.py:504-505)
    half_precision: bool = False

    @property
    def chunk_size(self) -> int:
        if self.all_negs:
            return self.batch_size
        if self.num_batch_negs > 0:
            return min(self.num_batch_negs, self.batch_size)
        return min(self.num_uniform_negs, self.batch_size)

    @property
    def num_chunks(self) -> int:
        return (self.batch_size - 1) // self.chunk_size + 1

    def num_negs(self, side_disabled: bool, num_rows: int = 0) -> int:
        """Negative columns of one side; with all_negs that is `num_rows`, the side's table size."""
        if side_disabled:
            return 0
        if self.all_negs:
            return num_rows
        return (self.chunk_size if self.num_batch_negs > 0 else 0) + self.num_uniform_negs


class StepRunner:
    """Owns the descriptor, the workspace and the output buffers of
    pbg_train_step / pbg_model_forward for one configuration and one pair of
    tables.  The tables, optimizer state and operator parameters are borrowed:
    the step updates them in place."""

    def __init__(self, spec: StepSpec, w_lhs: torch.Tensor, g_lhs: torch.Tensor,
                 w_rhs: Optional[torch.Tensor] = None, g_rhs: Optional[torch.Tensor] = None,
                 rhs_op: Optional[Dict[str, torch.Tensor]] = None, rhs_op_sum: Optional[Dict[str, torch.Tensor]] = None,
                 lhs_op: Optional[Dict[str, torch.Tensor]] = None, lhs_op_sum: Optional[Dict[str, torch.Tensor]] = None,
                 relation_weights: Optional[torch.Tensor] = None,
                 global_embs: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
                 global_sums: Optional[Tuple[torch.Tensor, torch.Tensor]] = None):
        """global_embs / global_sums: (lhs, rhs) global embedding [D] of each side's entity
        type and its AsyncAdagrad sum; the same tensor twice when the sides share a type."""
        self.spec = spec
        shared = w_rhs is None or w_rhs.data_ptr() == w_lhs.data_ptr()
        self.w_lhs = _need(w_lhs, torch.float32, "w_lhs")
        self.g_lhs = _need(g_lhs, torch.float32, "g_lhs")
        self.w_rhs = self.w_lhs if shared else _need(w_rhs, torch.float32, "w_rhs")
        self.g_rhs = self.g_lhs if shared else _need(g_rhs, torch.float32, "g_rhs")
        dev = w_lhs.device
        self.device = dev
        if spec.operator not in OPERATOR_CODES:
            raise NotImplementedError(f"Unknown operator {spec.operator}")
        if spec.comparator not in COMPARATOR_CODES:
            raise NotImplementedError(f"Unknown comparator {spec.comparator}")
        if spec.loss not in LOSS_CODES:
            raise NotImplementedError(f"Unknown loss {spec.loss}")
        d = StepDesc()
        d.dim = spec.dim
        d.num_workers = spec.num_workers
        d.batch_size = spec.batch_size
        d.num_batch_negs = spec.num_batch_negs
        d.num_uniform_negs = spec.num_uniform_negs
        d.disable_lhs_negs = int(spec.disable_lhs_negs)
        d.disable_rhs_negs = int(spec.disable_rhs_negs)
        d.op = OPERATOR_CODES[spec.operator]
        d.dynamic = int(spec.dynamic)
        d.num_relations = spec.num_relations
        d.comparator = COMPARATOR_CODES[spec.comparator]
        d.loss = LOSS_CODES[spec.loss]
        d.margin = spec.margin
        d.lr = spec.lr
        d.relation_lr = spec.relation_lr if spec.relation_lr is not None else spec.lr
        d.shared_table = int(shared)
        d.num_lhs_rows = self.w_lhs.shape[0]
        d.num_rhs_rows = self.w_rhs.shape[0]
        d.regularization_coef = spec.regularization_coef
        d.max_norm = float(spec.max_norm) if spec.max_norm else 0.0
        d.bias = int(bool(spec.bias))
        d.all_negs = int(bool(spec.all_negs))
        d.half_precision = int(bool(spec.half_precision))
        self.desc = d
        self.rhs_op = rhs_op or {}
        self.rhs_op_sum = rhs_op_sum or {}
        self.lhs_op = lhs_op or {}
        self.lhs_op_sum = lhs_op_sum or {}
        if global_embs is not None and spec.dynamic:
            raise RuntimeError("Cannot have global embs with dynamic rels")  # model.py:488-489
        self.global_embs = global_embs
        self.global_sums = global_sums
        self.relation_weights = (
            relation_weights if relation_weights is not None
            else torch.ones(spec.num_relations, dtype=torch.float32, device=dev)
        )
        nbytes = _lib.lib().pbg_train_step_workspace_bytes(ctypes.byref(d))
        if nbytes == 0:
            check(_lib.lib().pbg_model_forward(ctypes.byref(d), None, None, None, None, None, None))
        self.workspace = _workspace(nbytes, dev)
        k = spec.num_workers
        self.loss_out = torch.zeros(k, dtype=torch.float32, device=dev)
        self.violators_out = torch.zeros((k, 2), dtype=torch.int64, device=dev)
        self.reg_out = torch.zeros(k, dtype=torch.float32, device=dev)  # Stats.reg of each batch

    @staticmethod
    def _op_pair(params: Dict[str, torch.Tensor]) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor]]:
        if not params:
            return None, None
        # two-parameter operators: (first slot, second slot) of pbg_step_buffers
        for first, second in (("p0", "p1"), ("real", "imag"), ("linear_transformation", "translation")):
            if first in params and second in params:
                return params[first], params[second]
        (only,) = params.values()
        return only, None

    def _buffers(self, lhs, rhs, rel, uniform_lhs, uniform_rhs, edge_weight, uniform_seed=None) -> StepBuffers:
        s = self.spec
        k, b = s.num_workers, s.batch_size
        _need(lhs, torch.int64, "lhs")
        _need(rhs, torch.int64, "rhs")
        _need(rel, torch.int64, "rel")
        if lhs.numel() != k * b or rhs.numel() != k * b:
            raise ValueError(f"lhs / rhs must hold num_workers * batch_size = {k * b} entries")
        if rel.numel() != (k * b if s.dynamic else k):
            raise ValueError("rel must hold one entry per edge (dynamic) or per batch (standard)")
        c, u = s.num_chunks, (0 if s.all_negs else s.num_uniform_negs)
        if s.all_negs:
            uniform_lhs = uniform_rhs = uniform_seed = None  # the negatives are the tables' rows in order
        if uniform_seed is not None and (uniform_lhs is not None or uniform_rhs is not None):
            raise ValueError("pass uniform negatives or a seed to draw them with, not both")
        for name, t, off in (("uniform_lhs", uniform_lhs, s.disable_lhs_negs), ("uniform_rhs", uniform_rhs, s.disable_rhs_negs)):
            if u > 0 and not off and uniform_seed is None:
                if t is None:
                    raise ValueError(f"{name} is required (or uniform_seed, to draw the negatives in the step)")
                _need(t, torch.int64, name)
                if t.numel() != k * c * u:
                    raise ValueError(f"{name} must be [num_workers, num_chunks, num_uniform_negs] = [{k}, {c}, {u}]")
        bufs = StepBuffers()
        bufs.w_lhs, bufs.g_lhs = _ptr(self.w_lhs), _ptr(self.g_lhs)
        bufs.w_rhs, bufs.g_rhs = _ptr(self.w_rhs), _ptr(self.g_rhs)
        bufs.lhs, bufs.rhs, bufs.rel = _ptr(lhs), _ptr(rhs), _ptr(rel)
        bufs.uniform_lhs, bufs.uniform_rhs = _ptr(uniform_lhs), _ptr(uniform_rhs)
        if edge_weight is not None:  # EdgeList.weight (edgelist.py:51-95): one fp32 weight per edge
            _need(edge_weight, torch.float32, "edge_weight")
            if edge_weight.numel() != k * b:
                raise ValueError(f"edge_weight must hold num_workers * batch_size = {k * b} entries")
        bufs.edge_weight = _ptr(edge_weight)
        bufs.relation_weights = _ptr(self.relation_weights)
        p0, p1 = self._op_pair(self.rhs_op)
        s0, s1 = self._op_pair(self.rhs_op_sum)
        bufs.rhs_op_p0, bufs.rhs_op_p1, bufs.rhs_op_s0, bufs.rhs_op_s1 = _ptr(p0), _ptr(p1), _ptr(s0), _ptr(s1)
        p0, p1 = self._op_pair(self.lhs_op)
        s0, s1 = self._op_pair(self.lhs_op_sum)
        bufs.lhs_op_p0, bufs.lhs_op_p1, bufs.lhs_op_s0, bufs.lhs_op_s1 = _ptr(p0), _ptr(p1), _ptr(s0), _ptr(s1)
        bufs.loss_out, bufs.violators_out = _ptr(self.loss_out), _ptr(self.violators_out)
        bufs.reg_out = _ptr(self.reg_out)
        if self.global_embs is not None:
            bufs.lhs_global, bufs.rhs_global = (_ptr(_need(t, torch.float32, "global embedding")) for t in self.global_embs)
            if self.global_sums is not None:
                bufs.lhs_global_sum, bufs.rhs_global_sum = (_ptr(_need(t, torch.float32, "global embedding sum"))
                                                            for t in self.global_sums)
        bufs.workspace, bufs.workspace_bytes = _ptr(self.workspace), self.workspace.numel()
        bufs.sample_uniform = int(uniform_seed is not None)
        bufs.uniform_seed = (uniform_seed or 0) & (2**64 - 1)
        return bufs

    def train(self, lhs, rhs, rel, uniform_lhs=None, uniform_rhs=None, edge_weight=None, uniform_seed=None,
              check_ids: bool = False, stats_out=None) -> None:
        """One lock-step training step over num_workers batches; statistics land
        in self.loss_out / self.violators_out (device, no sync) or, with
        `stats_out = (loss[K] float32, violators[K, 2] int64)`, in the caller's
        tensors (a loop over many calls hands in rows of one buffer and reduces
        them once).  The uniform
        negatives are either given ([K, C, U] per side) or drawn inside the step
        from `uniform_seed` (sample_uniform_negatives shows which).

        The kernels clamp an id outside its table instead of failing.  With
        `check_ids` the ids are range-checked first (one reduction per array and
        one host synchronisation) and an IndexError is raised as F.embedding does
        in the reference (model.py:60-61)."""
        if check_ids:
            self._check_ids(lhs, rhs, rel, uniform_lhs, uniform_rhs)
        bufs = self._buffers(lhs, rhs, rel, uniform_lhs, uniform_rhs, edge_weight, uniform_seed)
        if stats_out is not None:
            loss, viol = stats_out
            k = self.spec.num_workers
            if _need(loss, torch.float32, "stats_out[0]").numel() != k or _need(viol, torch.int64, "stats_out[1]").numel() != 2 * k:
                raise ValueError(f"stats_out must be (loss[{k}], violators[{k}, 2])")
            bufs.loss_out, bufs.violators_out = _ptr(loss), _ptr(viol)
        check(_lib.lib().pbg_train_step(ctypes.byref(self.desc), ctypes.byref(bufs), _stream()))

    def _check_ids(self, lhs, rhs, rel, uniform_lhs, uniform_rhs) -> None:
        bounds = []
        for name, ids, limit in (("lhs", lhs, self.w_lhs.shape[0]), ("rhs", rhs, self.w_rhs.shape[0]),
                                 ("rel", rel, self.spec.num_relations), ("uniform_lhs", uniform_lhs, self.w_lhs.shape[0]),
                                 ("uniform_rhs", uniform_rhs, self.w_rhs.shape[0])):
            if ids is not None and ids.numel() > 0:
                lo, hi = torch.aminmax(ids)
                bounds.append((name, limit, lo, hi))
        if not bounds:
            return
        found = torch.stack([torch.stack((lo, hi)) for _, _, lo, hi in bounds]).tolist()
        for (name, limit, _, _), (lo, hi) in zip(bounds, found):
            if lo < 0 or hi >= limit:
                raise IndexError(f"{name}: index out of range ({lo if lo < 0 else hi} not in [0, {limit}))")

    def capture_train(self, lhs, rhs, rel, uniform_lhs=None, uniform_rhs=None, edge_weight=None) -> "torch.cuda.CUDAGraph":
        """Records one train() call into a HIP graph and returns it.  The tensors
        passed here become the graph's static inputs: write the next step's edges
        and negatives INTO them (copy_, randint(out=...)) and call replay().  The
        launch-bound single-batch step (about ten dependent kernels of a few
        microseconds each) is what this is for.  The step records kernels only (no
        memset nodes, no allocation), so a replay does exactly what the call did."""
        self.train(lhs, rhs, rel, uniform_lhs, uniform_rhs, edge_weight)  # first-call set-up must not be captured
        torch.cuda.current_stream(self.device).synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            self.train(lhs, rhs, rel, uniform_lhs, uniform_rhs, edge_weight)
        return graph

    STAGES = ("prep", "operator", "scores", "loss", "backward_dn", "backward_da", "rowback", "params", "sort", "update")

    @property
    def fused(self) -> bool:
        """True when the step runs as the single LDS-resident chunk kernel."""
        return bool(_lib.lib().pbg_train_step_is_fused(ctypes.byref(self.desc)))

    @property
    def route(self) -> str:
        """Which kernels the step runs: "staged", "fused" (one LDS-resident chunk
        kernel) or "stream" (positives in LDS, negatives streamed past them)."""
        code = _lib.lib().pbg_train_step_route(ctypes.byref(self.desc))
        if code < 0:  # an invalid descriptor: -1 must not read as the last name
            raise ValueError(_lib.lib().pbg_last_error().decode("utf-8", "replace") or "invalid step descriptor")
        return ("staged", "fused", "stream")[code]

    def train_profiled(self, lhs, rhs, rel, uniform_lhs=None, uniform_rhs=None, edge_weight=None,
                       uniform_seed=None) -> List[float]:
        """train() with HIP events between the stages; synchronises and returns
        the stage durations in milliseconds (order: StepRunner.STAGES)."""
        bufs = self._buffers(lhs, rhs, rel, uniform_lhs, uniform_rhs, edge_weight, uniform_seed)
        n = _lib.lib().pbg_train_step_num_stages()
        out = (ctypes.c_float * n)()
        check(_lib.lib().pbg_train_step_profile(ctypes.byref(self.desc), ctypes.byref(bufs), _stream(), out))
        return [float(x) for x in out]

    def ranks(self, lhs, rhs, rel, uniform_lhs=None, uniform_rhs=None, edge_weight=None, auc_samples: int = 0,
              auc_seed: int = 0):
        """What ranking evaluation needs of a forward pass, without the [K, B, N]
        score tensors (pbg_model_ranks): (lhs_pos[K,B], rhs_pos[K,B], lhs_rank[K,B],
        rhs_rank[K,B] -- 1 + negatives scoring at least as high, 0 for a side without
        negatives --, loss_edge[K,B] under spec.loss, auc_hits[2] or None)."""
        s = self.spec
        k, b = s.num_workers, s.batch_size
        bufs = self._buffers(lhs, rhs, rel, uniform_lhs, uniform_rhs, edge_weight)
        dev = self.device
        lhs_pos = torch.empty((k, b), dtype=torch.float32, device=dev)
        rhs_pos = torch.empty((k, b), dtype=torch.float32, device=dev)
        lhs_rank = torch.empty((k, b), dtype=torch.int64, device=dev)
        rhs_rank = torch.empty((k, b), dtype=torch.int64, device=dev)
        loss_edge = torch.empty((k, b), dtype=torch.float32, device=dev)
        hits = torch.empty(2, dtype=torch.int64, device=dev) if auc_samples > 0 else None
        check(_lib.lib().pbg_model_ranks(ctypes.byref(self.desc), ctypes.byref(bufs), _ptr(lhs_pos), _ptr(rhs_pos),
                                         _ptr(lhs_rank), _ptr(rhs_rank), _ptr(loss_edge), int(auc_samples),
                                         auc_seed & (2**64 - 1), _ptr(hits), _stream()))
        return lhs_pos, rhs_pos, lhs_rank, rhs_rank, loss_edge, hits

    def forward(self, lhs, rhs, rel, uniform_lhs=None, uniform_rhs=None):
        """Scores only: (lhs_pos[K,B], rhs_pos[K,B], lhs_neg[K,B,Nl], rhs_neg[K,B,Nr])."""
        s = self.spec
        k, b = s.num_workers, s.batch_size
        bufs = self._buffers(lhs, rhs, rel, uniform_lhs, uniform_rhs, None)
        dev = self.device
        nl = s.num_negs(s.disable_lhs_negs, self.w_lhs.shape[0])
        nr = s.num_negs(s.disable_rhs_negs, self.w_rhs.shape[0])
        lhs_pos = torch.empty((k, b), dtype=torch.float32, device=dev)
        rhs_pos = torch.empty((k, b), dtype=torch.float32, device=dev)
        lhs_neg = torch.empty((k, b, nl), dtype=torch.float32, device=dev)
        rhs_neg = torch.empty((k, b, nr), dtype=torch.float32, device=dev)
        check(_lib.lib().pbg_model_forward(ctypes.byref(self.desc), ctypes.byref(bufs), _ptr(lhs_pos), _ptr(rhs_pos),
                                           _ptr(lhs_neg) if nl else None, _ptr(rhs_neg) if nr else None, _stream()))
        return lhs_pos, rhs_pos, lhs_neg, rhs_neg
