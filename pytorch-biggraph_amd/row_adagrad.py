"""Row-wise Adagrad on embedding tables (reference: torchbiggraph/row_adagrad.py).

Same constructor, state layout (``state[p]["sum"]`` of shape ``[num_rows]``) and
``step`` contract as the reference; the arithmetic runs in libpbg_hip
(pbg_row_adagrad_sparse / pbg_row_adagrad_dense).
"""
import torch
from torch.optim import Optimizer

from . import native


class RowAdagrad(Optimizer):
    def __init__(self, params, lr=1e-2, lr_decay=0, weight_decay=0):
        assert lr_decay == 0, "lr_decay not currently supported."
        defaults = {"lr": lr, "lr_decay": lr_decay, "weight_decay": weight_decay}
        super().__init__(params, defaults)
        for group in self.param_groups:
            for p in group["params"]:
                if p.dim() != 2:
                    raise ValueError("RowAdagrad only works on 2D tensors")
                self.state[p]["sum"] = p.new_zeros((p.shape[0],))
        self._workspace = None

    def share_memory(self):
        for group in self.param_groups:
            for p in group["params"]:
                self.state[p]["sum"].share_memory_()

    def _ws(self, nbytes: int, device) -> torch.Tensor:
        if self._workspace is None or self._workspace.numel() < nbytes or self._workspace.device != device:
            self._workspace = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=device)
        return self._workspace

    @torch.no_grad()
    def step_rows(self, p: torch.Tensor, idx: torch.Tensor, grad_rows: torch.Tensor, lr=None) -> None:
        """Sparse step from an uncoalesced (index, gradient row) list; `grad_rows`
        is used as scratch."""
        if idx.numel() == 0:
            return
        group = next(g for g in self.param_groups if any(q is p for q in g["params"]))
        nbytes = native._lib.lib().pbg_row_adagrad_sparse_workspace_bytes(idx.shape[0])
        native.row_adagrad_sparse(p.data, self.state[p]["sum"], idx.contiguous(), grad_rows.contiguous(),
                                  group["lr"] if lr is None else lr, self._ws(nbytes, p.device))

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        for group in self.param_groups:
            for p in group["params"]:
                if p.grad is None:
                    continue
                grad = p.grad.data
                if group["weight_decay"] != 0:
                    if grad.is_sparse:
                        raise RuntimeError("weight_decay option is not compatible with sparse gradients ")
                    grad = grad.add(p.data, alpha=group["weight_decay"])
                if grad.is_sparse:
                    if grad._indices().numel() == 0:
                        continue
                    # duplicates are summed inside the kernel: no coalesce() needed;
                    # the values are cloned because the kernel sums in place
                    self.step_rows(p, grad._indices()[0], grad._values().clone(), group["lr"])
                else:
                    native.row_adagrad_dense(p.data, self.state[p]["sum"], grad.contiguous(), group["lr"])
        return loss
