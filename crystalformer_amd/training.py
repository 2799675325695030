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


def make_optimizer(model: nn.Module, lr: float = 5e-4, betas=(0.9, 0.98), weight_decay: float = 1e-5,
                   sch_decay: float = 4000.0,
                   capturable: bool = False) -> Tuple[optim.Optimizer, lr_scheduler.LambdaLR]:
    nodecay, decay = [], []
    for m in model.modules():
        if isinstance(m, (nn.BatchNorm1d, nn.LayerNorm, nn.SyncBatchNorm)):
            nodecay.extend(m.parameters(False))
        else:
            for name, param in m.named_parameters(recurse=False):
                (nodecay if "bias" in name else decay).append(param)
    assert sum(p.numel() for p in nodecay + decay) == sum(p.numel() for p in model.parameters())
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
