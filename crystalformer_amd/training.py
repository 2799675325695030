"""Plain-torch training step with the reference's optimiser settings
(models/regression.py:106-135 step, :211-269 parameter groups and schedule;
params/latticeformer/default.json:5-12 values): AdamW, betas (0.9, 0.98),
weight decay 1e-5 on everything but biases and norm layers, gradient-norm clip
1.0, learning rate lr * sqrt(4000 / (4000 + t)), L1 loss."""
from __future__ import annotations

from typing import Tuple

import torch
import torch.nn.functional as F
from torch import nn, optim
from torch.optim import lr_scheduler


def decay_groups(model: nn.Module):
    """(parameters without weight decay, parameters with): biases and norm layers are
    exempt (models/regression.py:217-232)."""
    nodecay, decay = [], []
    for m in model.modules():
        if isinstance(m, (nn.BatchNorm1d, nn.LayerNorm, nn.SyncBatchNorm)):
            nodecay.extend(m.parameters(False))
        else:
            for name, param in m.named_parameters(recurse=False):
                (nodecay if "bias" in name else decay).append(param)
    assert sum(p.numel() for p in nodecay + decay) == sum(p.numel() for p in model.parameters())
    return nodecay, decay


def make_optimizer(model: nn.Module, lr: float = 5e-4, betas=(0.9, 0.98), weight_decay: float = 1e-5,
                   sch_decay: float = 4000.0,
                   capturable: bool = False) -> Tuple[optim.Optimizer, lr_scheduler.LambdaLR]:
    nodecay, decay = decay_groups(model)
    groups = [{"params": nodecay}, {"params": decay, "weight_decay": weight_decay}] if weight_decay > 0 \
        else [{"params": list(model.parameters())}]
    opt = optim.AdamW(groups, lr=lr, betas=betas, weight_decay=0.0, capturable=capturable)
    sch = lr_scheduler.LambdaLR(opt, lambda t: (sch_decay / (sch_decay + t)) ** 0.5)
    return opt, sch


def training_step(model: nn.Module, batch, opt: optim.Optimizer, sch=None, clip_norm: float = 1.0) -> torch.Tensor:
    """zero_grad -> forward -> L1 loss -> backward -> clip -> step -> schedule."""
    opt.zero_grad()
    out = model(batch)
    loss = F.l1_loss(out[:, 0], batch.y, reduction="none").mean()
    loss.backward()
    if clip_norm > 0:
        nn.utils.clip_grad_norm_(model.parameters(), clip_norm)
    opt.step()
    if sch is not None:
        sch.step()
    return loss.detach()


class FusedAdamW:
    """Gradient-norm clip, AdamW and the inverse square-root schedule of
    :func:`make_optimizer` / :func:`training_step` as one device-side update
    (``cf_adamw_step``: two kinds of launch over all parameters instead of one
    element-wise launch per tensor and operation).  The step counter, the
    gradient norm and the learning rate of the last update live in ``state``
    (device, 3 floats), so a captured graph of ``step()`` advances the schedule by
    itself on every replay."""

    def __init__(self, model: nn.Module, lr: float = 5e-4, betas=(0.9, 0.98), eps: float = 1e-8,
                 weight_decay: float = 1e-5, sch_decay: float = 4000.0, clip_norm: float = 1.0):
        from . import ops
        nodecay, decay = decay_groups(model)
        pairs = [(p, 0.0) for p in nodecay] + [(p, float(weight_decay)) for p in decay]
        pairs = [(p, wd) for p, wd in pairs if p.requires_grad]
        if not pairs:
            raise ValueError("FusedAdamW: no trainable parameters")
        self.params = [p for p, _ in pairs]
        self.weight_decay = [wd for _, wd in pairs]
        for p in self.params:
            if not p.is_cuda or p.dtype != torch.float32 or not p.is_contiguous():
                raise ValueError("FusedAdamW: parameters must be contiguous float32 tensors on the GPU")
        self.lr, self.betas, self.eps, self.sch_decay, self.clip_norm = lr, betas, eps, sch_decay, clip_norm
        self.exp_avg = [torch.zeros_like(p) for p in self.params]
        self.exp_avg_sq = [torch.zeros_like(p) for p in self.params]
        self.state = torch.zeros(3, dtype=torch.float32, device=self.params[0].device)
        self._plan = ops.AdamWPlan(self.params, self.exp_avg, self.exp_avg_sq, self.weight_decay)

    def zero_grad(self, set_to_none: bool = True) -> None:
        for p in self.params:
            if p.grad is not None:
                if set_to_none:
                    p.grad = None
                else:
                    p.grad.zero_()

    def step(self) -> None:
        """Every parameter needs a gradient (the model's parameters all take part in the loss)."""
        from . import ops
        ops.adamw_step(self._plan, [p.grad for p in self.params], self.lr, self.sch_decay, self.betas[0],
                       self.betas[1], self.eps, self.clip_norm, self.state)

    def state_dict(self) -> dict:
        return {"state": self.state.clone(), "exp_avg": [t.clone() for t in self.exp_avg],
                "exp_avg_sq": [t.clone() for t in self.exp_avg_sq]}

    def load_state_dict(self, sd: dict) -> None:
        self.state.copy_(sd["state"])
        for dst, src in zip(self.exp_avg, sd["exp_avg"]):
            dst.copy_(src)
        for dst, src in zip(self.exp_avg_sq, sd["exp_avg_sq"]):
            dst.copy_(src)


def fused_training_step(model: nn.Module, batch, opt: "FusedAdamW", zero_grad: bool = True) -> torch.Tensor:
    """:func:`training_step` with the fused pieces, on any batch, launched eagerly: row-block
    linear Functions in the blocks, all linear layers' weight gradients from one grouped
    launch pair after the backward pass, clip + AdamW + schedule as one device-side update
    (``opt`` carries the clip norm and the schedule).  About a third of the time of the plain
    step, which is bound by the host side of some four hundred launches."""
    from . import hip_funcs
    if zero_grad:
        opt.zero_grad(set_to_none=True)
    previous = hip_funcs.USE_LINEAR_FUNCTION
    hip_funcs.USE_LINEAR_FUNCTION = True
    try:
        out = model(batch)
        if out.shape[1] == 1:
            loss = hip_funcs.L1MeanLossHIP.apply(out, batch.y.reshape(-1, 1))   # loss and its gradient in one launch
        else:
            loss = F.l1_loss(out[:, 0], batch.y, reduction="none").mean()
        with hip_funcs.deferred_weight_grads():           # all linear layers' weight gradients at the end
            loss.backward()
    finally:
        hip_funcs.USE_LINEAR_FUNCTION = previous
    opt.step()
    return loss.detach()
