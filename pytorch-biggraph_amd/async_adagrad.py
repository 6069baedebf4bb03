"""HOGWILD-tolerant Adagrad for the operator parameters (reference:
torchbiggraph/async_adagrad.py:19-87); the dense update runs in libpbg_hip."""
import torch
from torch.optim import Adagrad

from . import native


class AsyncAdagrad(Adagrad):
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
                grad = p.grad
                state = self.state[p]
                state["step"] += 1
                if group["weight_decay"] != 0:
                    if grad.is_sparse:
                        raise RuntimeError("weight_decay option is not compatible with sparse gradients")
                    grad = grad.add(p, alpha=group["weight_decay"])
                clr = group["lr"] / (1 + (float(state["step"]) - 1) * group["lr_decay"])
                if grad.is_sparse:
                    # element-wise Adagrad leaves entries with a zero gradient untouched,
                    # so the sparse branch equals the dense one on the densified gradient
                    grad = grad.to_dense()
                native.async_adagrad_dense(p.data, state["sum"], grad.contiguous(), clr, group["eps"])
        return loss
